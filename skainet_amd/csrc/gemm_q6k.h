// Q6_K prompt products behind the activation sources of the Q4_K one (internal to the library).
#pragma once
#include "common.h"

// True where skn_gemm_q6k_multi takes a matrix: rows of whole superblocks, the kernels that unpack the blocks
// themselves not switched off, sizes within the 32-bit offsets they use.
bool skn_gemm_q6k_direct_ok(const skn_ctx* ctx, int n, int k, int m);

// One activation pass (bf16 rows, fp32 rows, or fp32 rows with RMSNorm inside the pass) for one to three Q6_K matrices
// [n_i, k]; a matrix with `accumulate` set is added to its output by the store.  Every matrix must pass
// skn_gemm_q6k_direct_ok.
int skn_gemm_q6k_multi(skn_ctx* ctx, const skn_gemm_seg* segs, int nseg, int k, const skn_gemm_src& src, int m);
