// TEST INFRASTRUCTURE ONLY.
// C binding around the reference's own mask generator so that the Python tests can
// call the real reference code (util/random_mask.cc, compiled from where it lies
// under /root/reference) and compare the oracle's restatement against it.
// Declared here instead of including the reference header so that nothing of the
// reference is copied or needed at run time besides its compiled object.
#include <vector>
#include <cstring>

void random_mask(int nrow, int ncol, int brow, int bcol, float block_density,
                 int& nnzb, int& padded_nnzb, std::vector<int>& indptr, std::vector<int>& indices,
                 int block_divisor, int block_padding, unsigned seed);

extern "C" int ref_random_mask(int nrow, int ncol, int brow, int bcol, float density,
                               int divisor, int padding, unsigned seed,
                               int* nnzb_out, int* padded_out, int* indptr_out, int* indices_out, long indices_cap)
{
    std::vector<int> indptr, indices;
    int nnzb = 0, padded = 0;
    random_mask(nrow, ncol, brow, bcol, density, nnzb, padded, indptr, indices, divisor, padding, seed);
    *nnzb_out = nnzb;
    *padded_out = padded;
    if ((long)indices.size() > indices_cap) return -1;
    std::memcpy(indptr_out, indptr.data(), sizeof(int) * indptr.size());
    std::memcpy(indices_out, indices.data(), sizeof(int) * indices.size());
    return 0;
}
