// Two probe kernels that measure what this GPU gives a kernel at best: a streaming read of device memory and a
// loop of bf16 matrix instructions.  The benchmark reports its fractions of the roofline against these measured
// ceilings beside the published ones (the reference times its kernels the same way, warm-up then best of several
// runs with a sync before the clock stops: runtime/src/lib.rs:1550-1569).
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 probe_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float probe_f32x4;

// every thread reads 16-byte pieces a grid apart, eight loads in flight; the sink keeps the loads alive
__global__ void __launch_bounds__(256)
probe_stream_k(const uint4* __restrict__ buf, size_t n, unsigned* __restrict__ sink) {
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    uint4 acc = make_uint4(0, 0, 0, 0);
    for (; i + 7 * stride < n; i += 8 * stride) {
        uint4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = buf[i + j * stride];
#pragma unroll
        for (int j = 0; j < 8; j++) { acc.x ^= v[j].x; acc.y ^= v[j].y; acc.z ^= v[j].z; acc.w ^= v[j].w; }
    }
    for (; i < n; i += stride) { const uint4 v = buf[i]; acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w; }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = acc.x;      // practically never: the result is not wanted
}

extern "C" int tp_probe_stream(const void* buf, long bytes, void* sink, int blocks, void* stream) {
    TP_REQUIRE(buf && sink && bytes >= 16 && blocks > 0, "probe_stream: needs a buffer of at least 16 bytes, a sink and blocks");
    TP_REQUIRE((uintptr_t)buf % 16 == 0, "probe_stream: the buffer must be 16-byte aligned");
    probe_stream_k<<<blocks, 256, 0, (hipStream_t)stream>>>((const uint4*)buf, (size_t)bytes / 16, (unsigned*)sink);
    return tp_check_launch("probe_stream");
}

// every wave issues `iters` rounds of independent bf16 matrix instructions, 131,072 flop a round: eight
// v_mfma_f32_16x16x32_bf16 (kind 0) or four v_mfma_f32_32x32x16_bf16 (kind 1).  Block 0 also reports how many
// shader clocks and how many ticks of the constant 100 MHz clock its loop took: the shader clock under this load.
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float probe_f32x16;

template <int KIND>
__global__ void __launch_bounds__(256)
probe_mfma_k(int iters, float* __restrict__ sink, long long* __restrict__ clocks) {
    probe_bf16x8 a, b;
#pragma unroll
    for (int e = 0; e < 8; e++) { a[e] = (__bf16)(0.25f * (float)((threadIdx.x + e) & 7)); b[e] = (__bf16)(0.5f * (float)((threadIdx.x * 3 + e) & 3)); }
    const long long c0 = clock64(), w0 = wall_clock64();
    float t = 0.f;
    if (KIND == 0) {
        probe_f32x4 acc[8];
#pragma unroll
        for (int j = 0; j < 8; j++) acc[j] = (probe_f32x4){0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int j = 0; j < 8; j++) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[j], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 8; j++) t += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3];
    } else {
        probe_f32x16 acc[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[j][e] = 0.f;
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) t += acc[j][0] + acc[j][5] + acc[j][10] + acc[j][15];
    }
    if (t == -1.f) sink[0] = t;                                                // never: the sums are not negative
    if (blockIdx.x == 0 && threadIdx.x == 0 && clocks) { clocks[0] = clock64() - c0; clocks[1] = wall_clock64() - w0; }
}

// flop of one launch: blocks * 4 waves * iters * 131072
extern "C" int tp_probe_mfma(int kind, int iters, int blocks, void* sink, void* clocks, void* stream) {
    TP_REQUIRE(iters > 0 && blocks > 0 && sink, "probe_mfma: needs iterations, blocks and a sink");
    if (kind == 0) probe_mfma_k<0><<<blocks, 256, 0, (hipStream_t)stream>>>(iters, (float*)sink, (long long*)clocks);
    else if (kind == 1) probe_mfma_k<1><<<blocks, 256, 0, (hipStream_t)stream>>>(iters, (float*)sink, (long long*)clocks);
    else return tp_fail("probe_mfma: kind %d is neither 0 (16x16x32) nor 1 (32x32x16)", kind);
    return tp_check_launch("probe_mfma");
}
