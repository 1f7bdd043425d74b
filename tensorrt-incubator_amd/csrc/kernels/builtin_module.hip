// The built-in kernel module: every cluster kernel in one gfx950 code object, so
// the host side loads one module and resolves kernels by name.
#include "amax.hip"
#include "amax_scales.hip"
#include "qdq.hip"
#include "dynq.hip"
#include "dynq_rows.hip"
#include "nvfp4.hip"
#include "norm.hip"
#include "gemm_w8a8.hip"
#include "gemm_w4a16.hip"
#include "gemm_dense.hip"
#include "util.hip"
