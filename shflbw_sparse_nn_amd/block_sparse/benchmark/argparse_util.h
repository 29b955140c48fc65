// Command lines of the two benchmark programs.  Same options, defaults and complaints as the reference's
// parsers (block_sparse/benchmark/argparse_util.h:10-128 for SpMM, :130-263 for SpConv), so the sweep
// scripts written for it (scripts/benchmark/*.sh) drive these programs unchanged.  One extra switch,
// --one-tile, times a single entry of the operator table instead of every name for the block size.
#pragma once
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <sstream>
#include <string>

struct CommonArgs {
    float density = 0.f;
    unsigned seed = 2021; // the default of every run (argparse_util.h:31)
    int pattern_code = -1; // 0 = block, 1 = block-2in4 (accepted, no operator behind it - as in the reference)
    int block_sz = 0;
    bool row_permute = false;
    bool store_pattern = false, load_pattern = false;
    std::string store_path, load_path;
    bool one_tile = false;
};

struct SpmmArgs : CommonArgs {
    int m = 0, n = 0, k = 0;
};

struct SpconvArgs : CommonArgs {
    int B = 0, H = 0, W = 0, C = 0, F = 0, R = 0, S = 0, stride = 1;
};

namespace benchmark_args {

inline const char* common_usage()
{
    return "        --d [density between 0~1]\n"
           "        --sparsity-type [block/block-2in4] \n"
           "        --block-size [16/32/64/128] \n"
           "        Optional cmdline args: \n"
           "        --row-permute : run spmm with random row-permutation \n"
           "        --random: set a random seed. by default 2021 for every run.\n"
           "        --store-pattern [file]: store the random sparse pattern generated,\n"
           "        --load-pattern  [file]: load the random sparse pattern from file\n"
           "        --one-tile : time one entry of the operator table only\n\n";
}

// options shared by both programs; returns true when argv[i] was one of them
inline bool parse_common(int argc, const char** argv, int& i, CommonArgs& a)
{
    const bool has_value = i != argc - 1;
    if (!strcmp(argv[i], "--d") && has_value) {
        a.density = (float)atof(argv[i + 1]);
    } else if (!strcmp(argv[i], "--block-size") && has_value) {
        a.block_sz = atoi(argv[i + 1]);
    } else if (!strcmp(argv[i], "--sparsity-type") && has_value) {
        if (!strcmp(argv[i + 1], "block"))
            a.pattern_code = 0;
        else if (!strcmp(argv[i + 1], "block-2in4"))
            a.pattern_code = 1;
    } else if (!strcmp(argv[i], "--row-permute")) {
        a.row_permute = true;
    } else if (!strcmp(argv[i], "--random")) {
        a.seed = (unsigned)std::chrono::system_clock::now().time_since_epoch().count();
    } else if (!strcmp(argv[i], "--store-pattern") && has_value) {
        a.store_pattern = true;
        a.store_path = argv[i + 1];
    } else if (!strcmp(argv[i], "--load-pattern") && has_value) {
        a.load_pattern = true;
        a.load_path = argv[i + 1];
    } else if (!strcmp(argv[i], "--one-tile")) {
        a.one_tile = true;
    } else {
        return false;
    }
    return true;
}

[[noreturn]] inline void fail(const std::string& usage, const char* why, const std::string& log)
{
    std::cerr << usage << why << log;
    exit(EXIT_FAILURE);
}

inline void check_common(const CommonArgs& a, const std::string& usage, const std::string& log)
{
    if (a.load_pattern) { // argparse_util.h:75-80: announced, never implemented
        std::cerr << "load pattern not implemented.\n";
        exit(EXIT_FAILURE);
    }
    if (!((a.block_sz & (a.block_sz - 1)) == 0 && a.block_sz >= 16))
        fail(usage, "Unsupported block size. Choose in 16/32/64/128. \n", log);
    if (a.pattern_code == -1) fail(usage, "sparsity-pattern is not given or unsupported.\n", log);
}

} // namespace benchmark_args

inline SpmmArgs parseSpmmArgs(int argc, const char** argv, bool verbose = false)
{
    const std::string usage = std::string("\tRequired cmdline args:\n"
                                          "        --m [M]\n"
                                          "        --n [N]\n"
                                          "        --k [K]\n") +
                              benchmark_args::common_usage();
    SpmmArgs a;
    for (int i = 1; i < argc; ++i) {
        const bool has_value = i != argc - 1;
        if (!strcmp(argv[i], "--m") && has_value)
            a.m = atoi(argv[i + 1]);
        else if (!strcmp(argv[i], "--n") && has_value)
            a.n = atoi(argv[i + 1]);
        else if (!strcmp(argv[i], "--k") && has_value)
            a.k = atoi(argv[i + 1]);
        else
            benchmark_args::parse_common(argc, argv, i, a);
    }
    std::stringstream log;
    log << "\narguments: m = " << a.m << "\nn = " << a.n << "\nk = " << a.k << "\ndensity = " << a.density
        << "\nseed = " << a.seed << "\nblock-size = " << a.block_sz << " x 1"
        << "\nsparsity-pattern = " << a.pattern_code << "\nrow-permute ? " << a.row_permute;
    if (a.store_pattern) log << "\nstore path = " << a.store_path;
    log << "\n";
    if (!a.load_pattern && (a.m == 0 || a.n == 0 || a.k == 0 || a.density == 0.f))
        benchmark_args::fail(usage, "Forget to set m,n,k or density? \n", log.str());
    benchmark_args::check_common(a, usage, log.str());
    if (verbose) std::cerr << log.str();
    return a;
}

inline SpconvArgs parseSpconvArgs(int argc, const char** argv, bool verbose = false)
{
    const std::string usage = std::string("\tRequired cmdline args:\n"
                                          "        --B [B]\n"
                                          "        --H [H]\n"
                                          "        --W [W]\n"
                                          "        --C [C]\n"
                                          "        --F [F]\n"
                                          "        --R [R]\n"
                                          "        --S [S]\n"
                                          "        --stride [stride]\n") +
                              benchmark_args::common_usage();
    SpconvArgs a;
    for (int i = 1; i < argc; ++i) {
        const bool has_value = i != argc - 1;
        struct {
            const char* flag;
            int* dst;
        } ints[] = {{"--B", &a.B}, {"--H", &a.H}, {"--W", &a.W}, {"--C", &a.C},
                    {"--F", &a.F}, {"--R", &a.R}, {"--S", &a.S}, {"--stride", &a.stride}};
        bool hit = false;
        for (auto& o : ints)
            if (!strcmp(argv[i], o.flag) && has_value) {
                *o.dst = atoi(argv[i + 1]);
                hit = true;
            }
        if (!hit) benchmark_args::parse_common(argc, argv, i, a);
    }
    std::stringstream log;
    log << "\narguments: B = " << a.B << "\nH = " << a.H << "\nW = " << a.W << "\nC = " << a.C << "\nF = " << a.F
        << "\nR = " << a.R << "\nS = " << a.S << "\nstride = " << a.stride << "\ndensity = " << a.density
        << "\nseed = " << a.seed << "\nblock-size = " << a.block_sz << " x 1"
        << "\nsparsity-pattern = " << a.pattern_code << "\nrow-permute ? " << a.row_permute;
    if (a.store_pattern) log << "\nstore path = " << a.store_path;
    log << "\n";
    if (!a.load_pattern && (a.B == 0 || a.H == 0 || a.W == 0 || a.C == 0 || a.F == 0 || a.R == 0 || a.S == 0 ||
                            a.density == 0.f))
        benchmark_args::fail(usage, "Forget to set m,n,k or density\n", log.str());
    if (a.stride <= 0) benchmark_args::fail(usage, "Negative stride is not allowed.\n", log.str());
    benchmark_args::check_common(a, usage, log.str());
    if (verbose) std::cerr << log.str();
    return a;
}
