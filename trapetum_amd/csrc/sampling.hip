// Token choice on the device: argmax, repetition penalty, temperature / top-k / top-p sampling.
#include "common.h"

// ---- argmax: the smallest index among the largest values (strict '>' scan in the reference:
// runtime/src/lib.rs:1376-1380; device twin runtime/cuda/codebook_gemv.cu:548-591).  One block per row. ----
__global__ void __launch_bounds__(1024)
argmax_k(const float* __restrict__ logits, int V, int* __restrict__ out) {
    __shared__ float sval[16];
    __shared__ int sidx[16];
    const float* z = logits + (size_t)blockIdx.x * V;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float v = z[i];
        if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }      // NaN never wins
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { sval[wave] = bv; sidx[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); w++)
            if (sval[w] > bv || (sval[w] == bv && sidx[w] < bi)) { bv = sval[w]; bi = sidx[w]; }
        out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
    }
}

extern "C" int tp_argmax(const float* logits, int B, int V, int* out, void* stream) {
    TP_REQUIRE(B > 0 && V > 0, "argmax: empty shape B=%d V=%d", B, V);
    argmax_k<<<B, 1024, 0, (hipStream_t)stream>>>(logits, V, out);
    return tp_check_launch("argmax");
}
