// Matrix products of the kernel library: Y[M,N] = X[M,K] . W[N,K]^T with fp32 accumulation.
// W is a checkpoint matrix as stored ([out, in], row-major), X the step's rows.
#pragma once
#include "common.h"

enum { TP_EPI_NONE = 0, TP_EPI_SOFTCAP = 1, TP_EPI_GATED = 2 };
// steps of 64 k a wave of the 8-row kernel has in flight at once: four waves a block read a K of 2,304 in one round of loads
#define TP_R8_MAX_STEPS 9

struct GemmArgs {
    const void* x; const void* w; void* y;
    int in_dtype, out_dtype;
    int M, N, K;            // N counts rows of W (for a gated product: 2 * padded units)
    int epilogue; float cap;
    int units;              // gated: columns of the output (the feed-forward width)
    int act;                // gated: the gate's activation (TP_ACT_*)
    void* workspace; size_t workspace_bytes;
    int defer;              // split products: leave the K slices in the workspace [slices, M, N] for the consumer to add
    int algo;               // the caller's choice of kernel (0: none; see tp_linear)
    hipStream_t stream;
};

// the constants a kernel's epilogue takes: the cap, or the gate activation's two
static inline float2 epi_constants(const GemmArgs& a) {
    float2 e = make_float2(a.cap, 0.f);
    if (a.epilogue == TP_EPI_GATED) tp_gate_constants(a.act, &e.x, &e.y);
    return e;
}

// plain tiled kernel, any dtype and shape; one fixed summation order per output element
int gemm_simple_launch(const GemmArgs& a);
// bf16 on the matrix cores: rows <= 64 (streams W once), and large row counts (LDS-tiled)
bool gemm_skinny_supports(const GemmArgs& a);
size_t gemm_skinny_workspace(const GemmArgs& a);
int gemm_skinny_launch(const GemmArgs& a);
// bf16 by plain multiply-adds for one or two rows: X in registers, W streamed in contiguous kilobytes
bool gemv_supports(const GemmArgs& a);
size_t gemv_workspace(const GemmArgs& a);
int gemv_launch(const GemmArgs& a);
// bf16 on the matrix cores for three to eight rows: blocks of 8 rows of W, every load of a block in flight at once
bool gemm_rows8_supports(const GemmArgs& a);
size_t gemm_rows8_workspace(const GemmArgs& a);
int gemm_rows8_launch(const GemmArgs& a);
bool gemm_mfma_supports(const GemmArgs& a);
int gemm_mfma_splits(const GemmArgs& a);
int gemm_mfma_launch(const GemmArgs& a);
