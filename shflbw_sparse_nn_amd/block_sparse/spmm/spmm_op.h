#pragma once
#include "blockwise_op.h"
