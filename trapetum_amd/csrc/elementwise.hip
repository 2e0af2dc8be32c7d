// Row-wise kernels: embedding, norms fused with the residual add, row gather, RoPE + cache write,
// gated activation.  One block per row; statistics, angles and sums in fp32.
#include "common.h"
#include <type_traits>

#include "error_channel.h"

// ---- embedding: out[r] = table[token[r]] * scale (fp32).  Reference: host gather of a pre-scaled fp16
// row, runtime/src/lib.rs:4555, model/export_gemma.py:59-61. -----------------------------------------
template <typename T>
__global__ void embed_rows_k(const int* __restrict__ tokens, const T* __restrict__ table, float scale,
                             float* __restrict__ out, int D, int V) {
    const int r = blockIdx.x;
    int tok = tokens[r];
    const bool ok = tok >= 0 && tok < V;
    if (!ok) tok = 0;
    const T* src = table + (size_t)tok * D;
    float* dst = out + (size_t)r * D;
    for (int i = threadIdx.x; i < D; i += blockDim.x) dst[i] = ok ? ld_f32(src + i) * scale : __uint_as_float(0x7fc00000u);
}

extern "C" int tp_embed_rows(const int* tokens, const void* table, int dtype, float scale, float* out,
                             int M, int D, int V, void* stream) {
    TP_REQUIRE(M > 0 && D > 0 && V > 0, "embed_rows: empty shape M=%d D=%d V=%d", M, D, V);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TP_BF16) embed_rows_k<bf16_t><<<M, 256, 0, s>>>(tokens, (const bf16_t*)table, scale, out, D, V);
    else if (dtype == TP_F32) embed_rows_k<float><<<M, 256, 0, s>>>(tokens, (const float*)table, scale, out, D, V);
    else return tp_fail("embed_rows: unknown dtype %d", dtype);
    return tp_check_launch("embed_rows");
}

// ---- RMSNorm: out = x * rsqrt(mean(x^2) + eps) * gain.  runtime/cuda/codebook_gemv.cu:192-202 ---------
template <typename TI, typename TO>
__global__ void rms_norm_k(const TI* __restrict__ x, const float* __restrict__ gain, float eps,
                           TO* __restrict__ out, int D) {
    __shared__ float red[16];
    const TI* xr = x + (size_t)blockIdx.x * D;
    TO* orow = out + (size_t)blockIdx.x * D;
    float ss = 0.f;
    for (int i = threadIdx.x; i < D; i += blockDim.x) { float v = ld_f32(xr + i); ss += v * v; }
    ss = block_sum(ss, red);
    const float scale = rsqrtf(ss / (float)D + eps);
    for (int i = threadIdx.x; i < D; i += blockDim.x) st_f32(orow + i, (ld_f32(xr + i) * scale) * gain[i]);
}

// the same for rows of at most 256 * EPT elements: every element is read once and kept in registers
template <typename TI, typename TO, int EPT, int NTH>
__global__ void __launch_bounds__(NTH)
rms_norm_reg_k(const TI* __restrict__ x, const float* __restrict__ gain, float eps, TO* __restrict__ out, int D) {
    __shared__ float red[16];
    const TI* xr = x + (size_t)blockIdx.x * D;
    TO* orow = out + (size_t)blockIdx.x * D;
    float v[EPT], gn[EPT];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < EPT; j++) {
        const int i = threadIdx.x + j * NTH;
        v[j] = i < D ? ld_f32(xr + i) : 0.f;
        gn[j] = i < D ? gain[i] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < EPT; j++) ss += v[j] * v[j];
    ss = block_sum(ss, red);
    const float scale = rsqrtf(ss / (float)D + eps);
#pragma unroll
    for (int j = 0; j < EPT; j++) {
        const int i = threadIdx.x + j * NTH;
        if (i < D) st_f32(orow + i, (v[j] * scale) * gn[j]);
    }
}

template <typename TI, typename TO>
static void rms_norm_launch(const void* x, const float* gain, float eps, void* out, int M, int D, hipStream_t s) {
    if (D <= 256 * 2) rms_norm_reg_k<TI, TO, 2, 256><<<M, 256, 0, s>>>((const TI*)x, gain, eps, (TO*)out, D);
    else if (M <= 128 && D <= 1024 * 4) rms_norm_reg_k<TI, TO, 4, 1024><<<M, 1024, 0, s>>>((const TI*)x, gain, eps, (TO*)out, D);
    else if (D <= 256 * 4) rms_norm_reg_k<TI, TO, 4, 256><<<M, 256, 0, s>>>((const TI*)x, gain, eps, (TO*)out, D);
    else if (D <= 256 * 12) rms_norm_reg_k<TI, TO, 12, 256><<<M, 256, 0, s>>>((const TI*)x, gain, eps, (TO*)out, D);
    else if (D <= 1024 * 8) rms_norm_reg_k<TI, TO, 8, 1024><<<M, 1024, 0, s>>>((const TI*)x, gain, eps, (TO*)out, D);
    else rms_norm_k<TI, TO><<<M, 256, 0, s>>>((const TI*)x, gain, eps, (TO*)out, D);
}

extern "C" int tp_rms_norm(const void* x, int in_dtype, const float* gain, float eps, void* out, int out_dtype,
                           int M, int D, void* stream) {
    TP_REQUIRE(M > 0 && D > 0, "rms_norm: empty shape M=%d D=%d", M, D);
    hipStream_t s = (hipStream_t)stream;
    if (in_dtype == TP_F32 && out_dtype == TP_F32) rms_norm_launch<float, float>(x, gain, eps, out, M, D, s);
    else if (in_dtype == TP_F32 && out_dtype == TP_BF16) rms_norm_launch<float, bf16_t>(x, gain, eps, out, M, D, s);
    else if (in_dtype == TP_BF16 && out_dtype == TP_F32) rms_norm_launch<bf16_t, float>(x, gain, eps, out, M, D, s);
    else if (in_dtype == TP_BF16 && out_dtype == TP_BF16) rms_norm_launch<bf16_t, bf16_t>(x, gain, eps, out, M, D, s);
    else return tp_fail("rms_norm: unknown dtypes %d -> %d", in_dtype, out_dtype);
    return tp_check_launch("rms_norm");
}

// ---- stream += norm_post(rows) (or rows); out = norm_next(stream).  The reference runs rmsnorm, an add in
// fp32 and the next rmsnorm as three launches: runtime/src/lib.rs:4532-4535, cu:539-542. -----------------
template <typename T>
__global__ void add_rms_norm_k(float* __restrict__ stream, const T* __restrict__ rows,
                               const float* __restrict__ gain_post, float eps_post,
                               const float* __restrict__ gain_next, float eps_next,
                               T* __restrict__ out, int D) {
    __shared__ float red[16];
    float* sr = stream + (size_t)blockIdx.x * D;
    const T* ar = rows + (size_t)blockIdx.x * D;
    float scale_a = 1.f;
    if (gain_post) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < D; i += blockDim.x) { float v = ld_f32(ar + i); ss += v * v; }
        ss = block_sum(ss, red);
        scale_a = rsqrtf(ss / (float)D + eps_post);
    }
    float ss2 = 0.f;
    for (int i = threadIdx.x; i < D; i += blockDim.x) {
        float a = ld_f32(ar + i);
        if (gain_post) a = (a * scale_a) * gain_post[i];
        const float v = sr[i] + a;
        sr[i] = v;
        ss2 += v * v;
    }
    if (!gain_next) return;
    ss2 = block_sum(ss2, red);
    const float scale_s = rsqrtf(ss2 / (float)D + eps_next);
    T* orow = out + (size_t)blockIdx.x * D;
    for (int i = threadIdx.x; i < D; i += blockDim.x) st_f32(orow + i, (sr[i] * scale_s) * gain_next[i]);   // own writes
}

// TR: type of the rows (float when they arrive as n_slices K slices of a product, each `slice_stride`
// elements apart, added here in slice order); T: type of the normed output.
template <typename TR, typename T, int EPT, int NTH>
__global__ void __launch_bounds__(NTH)
add_rms_norm_reg_k(float* __restrict__ stream, const TR* __restrict__ rows, int n_slices, long slice_stride,
                   const float* __restrict__ gain_post, float eps_post,
                   const float* __restrict__ gain_next, float eps_next, T* __restrict__ out, int D) {
    __shared__ float red[16];
    float* sr = stream + (size_t)blockIdx.x * D;
    const TR* ar = rows + (size_t)blockIdx.x * D;
    float a[EPT], v[EPT], gp[EPT], gn[EPT];
#pragma unroll
    for (int j = 0; j < EPT; j++) {
        const int i = threadIdx.x + j * NTH;
        const bool ok = i < D;
        // K slices: four loads in flight at a time (a loop of load-then-add would pay one memory round trip per
        // slice), added in slice order; past the last slice the load repeats it and adds nothing
        const int ic = ok ? i : 0;
        float sum = n_slices == 1 ? ld_f32(ar + ic) : 0.f;
        for (int s0 = 0; s0 < n_slices && n_slices > 1; s0 += 4) {
            float t[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int sl = s0 + u < n_slices ? s0 + u : n_slices - 1;
                t[u] = ld_f32(ar + (size_t)sl * slice_stride + ic);
            }
#pragma unroll
            for (int u = 0; u < 4; u++) sum += s0 + u < n_slices ? t[u] : 0.f;
        }
        a[j] = ok ? sum : 0.f;
        v[j] = ok ? sr[i] : 0.f;
        gp[j] = (ok && gain_post) ? gain_post[i] : 1.f;
        gn[j] = (ok && gain_next) ? gain_next[i] : 0.f;
    }
    float scale_a = 1.f;
    if (gain_post) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < EPT; j++) ss += a[j] * a[j];
        ss = block_sum(ss, red);
        scale_a = rsqrtf(ss / (float)D + eps_post);
    }
    float ss2 = 0.f;
#pragma unroll
    for (int j = 0; j < EPT; j++) {
        const int i = threadIdx.x + j * NTH;
        float t = a[j];
        if (gain_post) t = (t * scale_a) * gp[j];
        v[j] += t;
        if (i < D) { sr[i] = v[j]; ss2 += v[j] * v[j]; }
    }
    if (!gain_next) return;
    ss2 = block_sum(ss2, red);
    const float scale_s = rsqrtf(ss2 / (float)D + eps_next);
    T* orow = out + (size_t)blockIdx.x * D;
#pragma unroll
    for (int j = 0; j < EPT; j++) {
        const int i = threadIdx.x + j * NTH;
        if (i < D) st_f32(orow + i, (v[j] * scale_s) * gn[j]);
    }
}

// The same for many rows, where the kernel is bound by the volume of its loads: a lane takes four neighbouring
// elements per load (16 bytes of float32, 8 of bf16), CPT such chunks NTH lanes apart.  Needs D % 4 == 0.
__device__ __forceinline__ void ld4(const float* p, float (&o)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    o[0] = t.x; o[1] = t.y; o[2] = t.z; o[3] = t.w;
}
__device__ __forceinline__ void ld4(const bf16_t* p, float (&o)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    o[0] = __uint_as_float(t.x << 16); o[1] = __uint_as_float(t.x & 0xffff0000u);
    o[2] = __uint_as_float(t.y << 16); o[3] = __uint_as_float(t.y & 0xffff0000u);
}
__device__ __forceinline__ void st4(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void st4(bf16_t* p, const float (&v)[4]) {
    uint2 t;
    t.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
    t.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
    *reinterpret_cast<uint2*>(p) = t;
}

template <typename TR, typename T, int CPT, int NTH>
__global__ void __launch_bounds__(NTH)
add_rms_norm_vec_k(float* __restrict__ stream, const TR* __restrict__ rows, int n_slices, long slice_stride,
                   const float* __restrict__ gain_post, float eps_post,
                   const float* __restrict__ gain_next, float eps_next, T* __restrict__ out, int D) {
    __shared__ float red[16], red_next[16];             // one for each of the two sums: no barrier between their uses
    float* sr = stream + (size_t)blockIdx.x * D;
    const TR* ar = rows + (size_t)blockIdx.x * D;
    float a[CPT][4], v[CPT][4], gp[CPT][4], gn[CPT][4];
#pragma unroll
    for (int j = 0; j < CPT; j++) {
        const int i = (threadIdx.x + j * NTH) * 4;
        const bool ok = i < D;
        const int ic = ok ? i : 0;                       // a chunk past the row reads the row's first and counts as zero
        // the stream, the gains and a group of slices are asked for together: a loop of load-then-add would pay one
        // trip to memory per slice.  Slices are added in slice order; past the last one the load repeats it and adds
        // nothing.  Groups of four; a row of one chunk a lane takes twelve at a time while more than four are left
        // (a product of few rows comes in up to sixteen slices).
        ld4(sr + ic, v[j]);
        if (gain_post) ld4(gain_post + ic, gp[j]);
        if (gain_next) ld4(gain_next + ic, gn[j]);
        ld4(ar + ic, a[j]);
        auto add_group = [&](int s0, auto width) {
            constexpr int W = decltype(width)::value;
            float t[W][4];
#pragma unroll
            for (int u = 0; u < W; u++) ld4(ar + (size_t)(s0 + u < n_slices ? s0 + u : n_slices - 1) * slice_stride + ic, t[u]);
#pragma unroll
            for (int u = 0; u < W; u++)
#pragma unroll
                for (int e = 0; e < 4; e++) a[j][e] += s0 + u < n_slices ? t[u][e] : 0.f;
        };
        int s0 = 1;
        if (CPT == 1)
            for (; s0 + 4 < n_slices; s0 += 12) add_group(s0, std::integral_constant<int, 12>());
        for (; s0 < n_slices; s0 += 4) add_group(s0, std::integral_constant<int, 4>());
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (!ok) { a[j][e] = 0.f; v[j][e] = 0.f; }
            if (!gain_post) gp[j][e] = 1.f;
        }
    }
    float scale_a = 1.f;
    if (gain_post) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < CPT; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) ss += a[j][e] * a[j][e];
        ss = block_sum_once(ss, red);
        scale_a = rsqrtf(ss / (float)D + eps_post);
    }
    float ss2 = 0.f;
#pragma unroll
    for (int j = 0; j < CPT; j++) {
        const int i = (threadIdx.x + j * NTH) * 4;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float t = a[j][e];
            if (gain_post) t = (t * scale_a) * gp[j][e];
            v[j][e] += t;
            ss2 += v[j][e] * v[j][e];                    // chunks past the row hold zeros
        }
        if (i < D) st4(sr + i, v[j]);
    }
    if (!gain_next) return;
    ss2 = block_sum_once(ss2, red_next);
    const float scale_s = rsqrtf(ss2 / (float)D + eps_next);
    T* orow = out + (size_t)blockIdx.x * D;
#pragma unroll
    for (int j = 0; j < CPT; j++) {
        const int i = (threadIdx.x + j * NTH) * 4;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = (v[j][e] * scale_s) * gn[j][e];
        if (i < D) st4(orow + i, o);
    }
}

template <typename TR, typename T>
static int add_rms_norm_launch(float* stream, const void* rows, int n_slices, long slice_stride, const float* gp, float ep,
                               const float* gn, float en, void* out, int M, int D, hipStream_t s) {
    // few rows: many threads per row (the kernel is bound by the latency of its loads, not by their volume)
    // few rows: a chunk a lane and as many lanes as the row has chunks (the kernel is bound by the latency of its loads:
    // one 16-byte load per operand and lane; 2B decode of 64 sequences 3.51 -> 3.21 ms a step against 1,024 lanes of
    // four single elements)
    const bool aligned = D % 4 == 0 && (uintptr_t)rows % 16 == 0 && (uintptr_t)stream % 16 == 0 && slice_stride % 4 == 0 &&
                         (!gp || (uintptr_t)gp % 16 == 0) && (!gn || (uintptr_t)gn % 16 == 0) && (!out || (uintptr_t)out % 16 == 0);
    const bool few = aligned && M <= 128, vec = aligned && M > 128;
    // (HipOps.add_rms_norm adds the slices itself, with sum_slices, before it comes here with a wider row)
#define TP_ADD_NORM_VEC(CPT, NTH) add_rms_norm_vec_k<TR, T, CPT, NTH><<<M, NTH, 0, s>>>(stream, (const TR*)rows, n_slices, slice_stride, gp, ep, gn, en, (T*)out, D)
    if (few && D > 256 * 4 && D <= 640 * 4) TP_ADD_NORM_VEC(1, 640);
    else if (few && D > 640 * 4 && D <= 1024 * 4) TP_ADD_NORM_VEC(1, 1024);
    else if (few && D > 1024 * 4 && D <= 640 * 8) TP_ADD_NORM_VEC(2, 640);
    else if (few && D > 640 * 8 && D <= 1024 * 8) TP_ADD_NORM_VEC(2, 1024);
    else if (vec && D <= 256 * 4) TP_ADD_NORM_VEC(1, 256);
    // many rows: three chunks a lane and just the waves that fills (a width of 2,304 is 576 chunks: three waves a
    // block, so that the CUs hold every block of 2,048 rows at once and no lane idles; 256 lanes left a quarter of
    // them idle and the last quarter of the blocks waiting)
    else if (vec && D <= 128 * 12) TP_ADD_NORM_VEC(3, 128);
    else if (vec && D <= 192 * 12) TP_ADD_NORM_VEC(3, 192);
    else if (vec && D <= 256 * 12) TP_ADD_NORM_VEC(3, 256);
    else if (vec && D <= 320 * 12) TP_ADD_NORM_VEC(3, 320);
    else if (vec && D <= 384 * 12) TP_ADD_NORM_VEC(3, 384);
    else if (vec && D <= 448 * 12) TP_ADD_NORM_VEC(3, 448);
    else if (vec && D <= 512 * 12) TP_ADD_NORM_VEC(3, 512);
    else if (vec && D <= 512 * 16) TP_ADD_NORM_VEC(4, 512);
    else if (D <= 256 * 2) add_rms_norm_reg_k<TR, T, 2, 256><<<M, 256, 0, s>>>(stream, (const TR*)rows, n_slices, slice_stride, gp, ep, gn, en, (T*)out, D);
    else if (M <= 128 && D <= 1024 * 4) add_rms_norm_reg_k<TR, T, 4, 1024><<<M, 1024, 0, s>>>(stream, (const TR*)rows, n_slices, slice_stride, gp, ep, gn, en, (T*)out, D);
    else if (D <= 256 * 4) add_rms_norm_reg_k<TR, T, 4, 256><<<M, 256, 0, s>>>(stream, (const TR*)rows, n_slices, slice_stride, gp, ep, gn, en, (T*)out, D);
    else if (D <= 256 * 12) add_rms_norm_reg_k<TR, T, 12, 256><<<M, 256, 0, s>>>(stream, (const TR*)rows, n_slices, slice_stride, gp, ep, gn, en, (T*)out, D);
    else if (D <= 1024 * 8) add_rms_norm_reg_k<TR, T, 8, 1024><<<M, 1024, 0, s>>>(stream, (const TR*)rows, n_slices, slice_stride, gp, ep, gn, en, (T*)out, D);
    else if (n_slices == 1 && sizeof(TR) == sizeof(T)) add_rms_norm_k<T><<<M, 256, 0, s>>>(stream, (const T*)rows, gp, ep, gn, en, (T*)out, D);
    else return tp_fail("add_rms_norm: rows in slices need a width of at most %d, found %d", 1024 * 8, D);
#undef TP_ADD_NORM_VEC
    return 0;
}

extern "C" int tp_add_rms_norm(float* stream, const void* rows, int rows_dtype, int n_slices, long slice_stride,
                               const float* gain_post, float eps_post, const float* gain_next, float eps_next,
                               void* out, int out_dtype, int M, int D, void* stream_) {
    TP_REQUIRE(M > 0 && D > 0, "add_rms_norm: empty shape M=%d D=%d", M, D);
    TP_REQUIRE(!gain_next || out, "add_rms_norm: a next norm needs an output buffer");
    TP_REQUIRE(n_slices >= 1 && (n_slices == 1 || rows_dtype == TP_F32), "add_rms_norm: rows in %d slices must be float32", n_slices);
    hipStream_t s = (hipStream_t)stream_;
    int rc;
    if (rows_dtype == TP_BF16 && out_dtype == TP_BF16) rc = add_rms_norm_launch<bf16_t, bf16_t>(stream, rows, n_slices, slice_stride, gain_post, eps_post, gain_next, eps_next, out, M, D, s);
    else if (rows_dtype == TP_F32 && out_dtype == TP_F32) rc = add_rms_norm_launch<float, float>(stream, rows, n_slices, slice_stride, gain_post, eps_post, gain_next, eps_next, out, M, D, s);
    else if (rows_dtype == TP_F32 && out_dtype == TP_BF16) rc = add_rms_norm_launch<float, bf16_t>(stream, rows, n_slices, slice_stride, gain_post, eps_post, gain_next, eps_next, out, M, D, s);
    else return tp_fail("add_rms_norm: unsupported dtypes rows %d -> out %d", rows_dtype, out_dtype);
    if (rc) return rc;
    return tp_check_launch("add_rms_norm");
}

// ---- the K slices of a product added in slice order (for a consumer that does not add them itself) --------------
template <typename T>
__global__ void sum_slices_k(const float* __restrict__ slices, int n_slices, long slice_stride, T* __restrict__ out, long count) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (long)gridDim.x * blockDim.x) {
        float t = 0.f;
        for (int s = 0; s < n_slices; s++) t += slices[(size_t)s * slice_stride + i];
        st_f32(out + i, t);
    }
}

extern "C" int tp_sum_slices(const float* slices, int n_slices, long slice_stride, void* out, int out_dtype, long count, void* stream) {
    TP_REQUIRE(slices && out && n_slices >= 1 && count > 0 && slice_stride >= count, "sum_slices: %d slices of %ld elements, %ld apart", n_slices, count, slice_stride);
    const int blocks = (int)((count + 255) / 256 < 4096 ? (count + 255) / 256 : 4096);
    if (out_dtype == TP_BF16) sum_slices_k<bf16_t><<<blocks, 256, 0, (hipStream_t)stream>>>(slices, n_slices, slice_stride, (bf16_t*)out, count);
    else if (out_dtype == TP_F32) sum_slices_k<float><<<blocks, 256, 0, (hipStream_t)stream>>>(slices, n_slices, slice_stride, (float*)out, count);
    else return tp_fail("sum_slices: unknown dtype %d", out_dtype);
    return tp_check_launch("sum_slices");
}

// ---- gather rows of the fp32 stream -------------------------------------------------------------------
__global__ void gather_rows_k(const float* __restrict__ x, const int* __restrict__ rows, float* __restrict__ out, int D, int M) {
    int r = rows[blockIdx.x];
    r = r < 0 ? 0 : (r >= M ? M - 1 : r);
    const float* src = x + (size_t)r * D;
    float* dst = out + (size_t)blockIdx.x * D;
    for (int i = threadIdx.x; i < D; i += blockDim.x) dst[i] = src[i];
}

extern "C" int tp_gather_rows(const float* x, const int* rows, float* out, int n, int D, int M, void* stream) {
    TP_REQUIRE(n > 0 && D > 0 && M > 0, "gather_rows: empty shape n=%d D=%d M=%d", n, D, M);
    gather_rows_k<<<n, 256, 0, (hipStream_t)stream>>>(x, rows, out, D, M);
    return tp_check_launch("gather_rows");
}

// ---- RoPE on q and k in place, then k and v into the paged cache -----------------------------------------
// Rotation: pair (d, d + rot/2), angle = pos * inv_freq[d], fp32 cos/sin (runtime/cuda/codebook_gemv.cu:219-230);
// the cache keeps k after the rotation and v as projected (runtime/src/lib.rs:4487-4490).
// A sequence's position p lives in row p (or p % rows_cap of a ring), found through its page list.
// grid (rows, groups of heads): a block rotates `hpb` of the row's H + KV heads (query heads first); a thread
// computes the cosine and sine of its pair once and applies them to all of them.  A key head goes into the
// cache, with its value head, straight from registers; without a page table the keys are rotated and nothing is
// cached (a step whose attention still has to read the cache as earlier steps left it caches its rows afterwards).
template <typename T>
__global__ void __launch_bounds__(128)
rope_kv_write_k(T* __restrict__ q, long q_stride, T* __restrict__ k, long k_stride,
                const T* __restrict__ v, long v_stride, int H, int KV, int hd,
                const float* __restrict__ inv_freq, int rot,
                const int* __restrict__ row_seq, const int* __restrict__ row_pos,
                const int* __restrict__ new_len, const int* __restrict__ table, int table_w,
                T* __restrict__ k_pool, T* __restrict__ v_pool, int page, int rows_cap, int hpb, int pairing) {
    const int r = blockIdx.x;
    const int j_begin = blockIdx.y * hpb, j_end = min(j_begin + hpb, H + (k ? KV : 0));
    const int pos = row_pos[r];
    const int half = rot / 2;
    // where the row's keys and values go: the same page and row for every kv head
    size_t cache_at = 0;
    bool cached = false;
    if (k && table && j_end > H) {
        const int seq = row_seq[r];
        int row = pos;
        bool keep = true;
        if (rows_cap > 0) {
            keep = pos + rows_cap >= new_len[seq];       // else a later row of this step takes the same ring row
            row = pos % rows_cap;
        }
        const int pg = keep ? table[(size_t)seq * table_w + row / page] : -1;
        cached = pg >= 0;
        if (cached) cache_at = ((size_t)pg * KV * page + row % page) * hd;      // + kv head * page * hd
    }
    for (int f = threadIdx.x; f < half; f += blockDim.x) {     // one thread per pair: elements (f, f + half), or neighbours (2f, 2f + 1)
        const float ang = (float)pos * inv_freq[f];
        const float c = cosf(ang), sn = sinf(ang);
        const int e0 = pairing == TP_ROPE_NEIGHBOURS ? 2 * f : f, e1 = pairing == TP_ROPE_NEIGHBOURS ? 2 * f + 1 : f + half;
        for (int j = j_begin; j < j_end; j++) {
            const bool is_q = j < H;
            T* x = is_q ? q + (size_t)r * q_stride + (size_t)j * hd : k + (size_t)r * k_stride + (size_t)(j - H) * hd;
            const float x0 = ld_f32(x + e0), x1 = ld_f32(x + e1);
            const float y0 = x0 * c - x1 * sn, y1 = x1 * c + x0 * sn;
            st_f32(x + e0, y0);
            st_f32(x + e1, y1);
            if (is_q) continue;
            const T* vsrc = v + (size_t)r * v_stride + (size_t)(j - H) * hd;
            if (cached) {
                const size_t off = cache_at + (size_t)(j - H) * page * hd;
                st_f32(k_pool + off + e0, y0);
                st_f32(k_pool + off + e1, y1);
                v_pool[off + e0] = vsrc[e0];
                v_pool[off + e1] = vsrc[e1];
            }
        }
    }
    if (cached)
        for (int j = max(j_begin, H); j < j_end; j++) {           // elements outside the rotation
            const size_t off = cache_at + (size_t)(j - H) * page * hd;
            const T* ksrc = k + (size_t)r * k_stride + (size_t)(j - H) * hd;
            const T* vsrc = v + (size_t)r * v_stride + (size_t)(j - H) * hd;
            for (int d = rot + threadIdx.x; d < hd; d += blockDim.x) { k_pool[off + d] = ksrc[d]; v_pool[off + d] = vsrc[d]; }
        }
}

// The same for many bf16 rows of heads whose rotated half is whole 16-byte pieces: a block per row works out the
// row's cosines and sines once into LDS, then every thread turns 8 pairs of one head with two 16-byte loads and
// stores (the 2B prefills of the benchmark, 2,048 and 4,096 rows: 18.5 -> 12.9 us a layer on average).
__global__ void __launch_bounds__(256)
rope_kv_write_vec_k(bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ k, long k_stride,
                    const bf16_t* __restrict__ v, long v_stride, int H, int KV, int hd,
                    const float* __restrict__ inv_freq, int rot,
                    const int* __restrict__ row_seq, const int* __restrict__ row_pos,
                    const int* __restrict__ new_len, const int* __restrict__ table, int table_w,
                    bf16_t* __restrict__ k_pool, bf16_t* __restrict__ v_pool, int page, int rows_cap) {
    // cosine and sine of pair f at [f % 8][f / 8]: the threads of a wave, which turn neighbouring pieces of 8 pairs, then
    // read neighbouring words (pair by pair in the pairs' own order, a wave's reads fell on four banks)
    __shared__ float cs[8 * 16], sn[8 * 16];
    const int r = blockIdx.x, pos = row_pos[r], half = rot / 2;
    for (int f = threadIdx.x; f < half; f += 256) {
        const float ang = (float)pos * inv_freq[f];
        cs[(f & 7) * 16 + (f >> 3)] = cosf(ang);
        sn[(f & 7) * 16 + (f >> 3)] = sinf(ang);
    }
    size_t cache_at = 0;
    bool cached = false;
    if (k && table) {
        const int seq = row_seq[r];
        int row = pos;
        bool keep = true;
        if (rows_cap > 0) {
            keep = pos + rows_cap >= new_len[seq];       // else a later row of this step takes the same ring row
            row = pos % rows_cap;
        }
        const int pg = keep ? table[(size_t)seq * table_w + row / page] : -1;
        cached = pg >= 0;
        if (cached) cache_at = ((size_t)pg * KV * page + row % page) * hd;      // + kv head * page * hd
    }
    __syncthreads();
    union Piece { uint4 u; bf16_t h[8]; };
    const int pieces = half / 8, heads = H + (k ? KV : 0);
    for (int item = threadIdx.x; item < heads * pieces; item += 256) {
        const int j = item / pieces, piece = item - j * pieces, f0 = piece * 8;
        const bool is_q = j < H;
        bf16_t* x = is_q ? q + (size_t)r * q_stride + (size_t)j * hd : k + (size_t)r * k_stride + (size_t)(j - H) * hd;
        Piece lo, hi;
        lo.u = *reinterpret_cast<const uint4*>(x + f0);
        hi.u = *reinterpret_cast<const uint4*>(x + f0 + half);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float x0 = bf16_to_f32(lo.h[e]), x1 = bf16_to_f32(hi.h[e]), c = cs[e * 16 + piece], sv = sn[e * 16 + piece];
            lo.h[e] = f32_to_bf16(x0 * c - x1 * sv);
            hi.h[e] = f32_to_bf16(x1 * c + x0 * sv);
        }
        *reinterpret_cast<uint4*>(x + f0) = lo.u;
        *reinterpret_cast<uint4*>(x + f0 + half) = hi.u;
        if (is_q) continue;
        const bf16_t* vsrc = v + (size_t)r * v_stride + (size_t)(j - H) * hd;
        const uint4 v0 = *reinterpret_cast<const uint4*>(vsrc + f0), v1 = *reinterpret_cast<const uint4*>(vsrc + f0 + half);
        if (cached) {
            const size_t off = cache_at + (size_t)(j - H) * page * hd;
            *reinterpret_cast<uint4*>(k_pool + off + f0) = lo.u;
            *reinterpret_cast<uint4*>(k_pool + off + f0 + half) = hi.u;
            *reinterpret_cast<uint4*>(v_pool + off + f0) = v0;
            *reinterpret_cast<uint4*>(v_pool + off + f0 + half) = v1;
        }
    }
    if (cached) {                                                 // elements outside the rotation
        const int rest = (hd - rot) / 8;
        for (int item = threadIdx.x; item < KV * rest; item += 256) {
            const int j = item / rest, d = rot + (item - j * rest) * 8;
            const uint4 kk = *reinterpret_cast<const uint4*>(k + (size_t)r * k_stride + (size_t)j * hd + d);
            const uint4 vv = *reinterpret_cast<const uint4*>(v + (size_t)r * v_stride + (size_t)j * hd + d);
            const size_t off = cache_at + (size_t)j * page * hd + d;
            *reinterpret_cast<uint4*>(k_pool + off) = kk;
            *reinterpret_cast<uint4*>(v_pool + off) = vv;
        }
    }
}

extern "C" int tp_rope_kv_write(void* q, long q_stride, void* k, long k_stride, const void* v, long v_stride,
                                int dtype, int M, int H, int KV, int hd, const float* inv_freq, int rot,
                                const int* row_seq, const int* row_pos, const int* new_len,
                                const int* table, int table_w, void* k_pool, void* v_pool,
                                int page, int rows_cap, int pairing, void* stream) {
    TP_REQUIRE(M > 0 && H > 0 && hd > 0, "rope_kv_write: empty shape M=%d H=%d hd=%d", M, H, hd);
    TP_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0, "rope_kv_write: rotary_dim %d must be even and at most head_dim %d", rot, hd);
    TP_REQUIRE(rot == 0 || inv_freq, "rope_kv_write: a rotation needs its frequency table");
    TP_REQUIRE(pairing == TP_ROPE_HALVES || pairing == TP_ROPE_NEIGHBOURS, "rope_kv_write: pairing %d is neither halves (%d) nor neighbours (%d)",
               pairing, TP_ROPE_HALVES, TP_ROPE_NEIGHBOURS);
    // table null: the keys are rotated and nothing is cached
    TP_REQUIRE(!k || (v && KV > 0), "rope_kv_write: keys without values");
    TP_REQUIRE(!k || !table || (k_pool && v_pool && page > 0 && table_w > 0), "rope_kv_write: a page table without cache pools");
    if (!table) { page = 1; rows_cap = 0; }
    TP_REQUIRE(rows_cap >= 0 && (rows_cap == 0 || rows_cap % page == 0), "rope_kv_write: ring of %d rows is no multiple of the page size %d", rows_cap, page);
    hipStream_t s = (hipStream_t)stream;
    TP_REQUIRE(H + KV <= 65535, "rope_kv_write: %d heads exceed one launch", H + KV);
    const int heads = H + (k ? KV : 0);
    auto piecewise = [](const void* p, long stride) { return !p || ((uintptr_t)p % 16 == 0 && stride % 8 == 0); };
    if (pairing == TP_ROPE_HALVES && dtype == TP_BF16 && M >= 256 && hd % 8 == 0 && rot % 16 == 0 && rot <= 256 && piecewise(q, q_stride) && piecewise(k, k_stride) &&
        piecewise(v, v_stride) && piecewise(k_pool, 8) && piecewise(v_pool, 8)) {
        rope_kv_write_vec_k<<<M, 256, 0, s>>>((bf16_t*)q, q_stride, (bf16_t*)k, k_stride, (const bf16_t*)v, v_stride, H, KV, hd,
            inv_freq, rot, row_seq, row_pos, new_len, table, table_w, (bf16_t*)k_pool, (bf16_t*)v_pool, page, rows_cap);
        return tp_check_launch("rope_kv_write");
    }
    // many rows: one block per row shares each pair's cosine and sine over all heads; few rows: a block per head
    const int hpb = M >= 256 ? heads : (M >= 32 ? (heads + 3) / 4 : 1);
    dim3 grid(M, (heads + hpb - 1) / hpb);
    const int threads = hd <= 64 ? 64 : 128;
    if (dtype == TP_BF16)
        rope_kv_write_k<bf16_t><<<grid, threads, 0, s>>>((bf16_t*)q, q_stride, (bf16_t*)k, k_stride, (const bf16_t*)v, v_stride, H, KV, hd,
            inv_freq, rot, row_seq, row_pos, new_len, table, table_w, (bf16_t*)k_pool, (bf16_t*)v_pool, page, rows_cap, hpb, pairing);
    else if (dtype == TP_F32)
        rope_kv_write_k<float><<<grid, threads, 0, s>>>((float*)q, q_stride, (float*)k, k_stride, (const float*)v, v_stride, H, KV, hd,
            inv_freq, rot, row_seq, row_pos, new_len, table, table_w, (float*)k_pool, (float*)v_pool, page, rows_cap, hpb, pairing);
    else return tp_fail("rope_kv_write: unknown dtype %d", dtype);
    return tp_check_launch("rope_kv_write");
}

// ---- a step's keys (rotated already) and values into the paged cache ------------------------------------------------
// For steps whose attention reads the cache as earlier steps left it and therefore caches its own rows afterwards: in a
// ring without a row to spare the step's rows take the places of positions that its earlier queries still see.
// grid (rows); a block copies the row's kv heads of K and V; of rows that share a ring row the last one stays.
template <typename T>
__global__ void __launch_bounds__(256)
kv_write_k(const T* __restrict__ k, long k_stride, const T* __restrict__ v, long v_stride, int KV, int hd,
           const int* __restrict__ row_seq, const int* __restrict__ row_pos, const int* __restrict__ new_len,
           const int* __restrict__ table, int table_w, T* __restrict__ k_pool, T* __restrict__ v_pool, int page, int rows_cap) {
    const int r = blockIdx.x, seq = row_seq[r], pos = row_pos[r];
    int row = pos;
    if (rows_cap > 0) {
        if (pos + rows_cap < new_len[seq]) return;       // a later row of this step takes the same ring row
        row = pos % rows_cap;
    }
    const int pg = table[(size_t)seq * table_w + row / page];
    if (pg < 0) return;                                  // never for a position the cache has room for
    const size_t at = ((size_t)pg * KV * page + row % page) * hd;
    constexpr int PIECE = 16 / sizeof(T);                // elements of a 16-byte piece
    const bool wide = hd % PIECE == 0 && k_stride % PIECE == 0 && v_stride % PIECE == 0 && (uintptr_t)k % 16 == 0 &&
                      (uintptr_t)v % 16 == 0 && (uintptr_t)k_pool % 16 == 0 && (uintptr_t)v_pool % 16 == 0;
    if (wide) {
        const int per_head = hd / PIECE;
        for (int i = threadIdx.x; i < KV * per_head; i += blockDim.x) {
            const int g = i / per_head, d = (i - g * per_head) * PIECE;
            const size_t dst = at + (size_t)g * page * hd + d;
            *reinterpret_cast<uint4*>(k_pool + dst) = *reinterpret_cast<const uint4*>(k + (size_t)r * k_stride + (size_t)g * hd + d);
            *reinterpret_cast<uint4*>(v_pool + dst) = *reinterpret_cast<const uint4*>(v + (size_t)r * v_stride + (size_t)g * hd + d);
        }
    } else {
        for (int i = threadIdx.x; i < KV * hd; i += blockDim.x) {
            const int g = i / hd, d = i - g * hd;
            const size_t dst = at + (size_t)g * page * hd + d;
            k_pool[dst] = k[(size_t)r * k_stride + i];
            v_pool[dst] = v[(size_t)r * v_stride + i];
        }
    }
}

extern "C" int tp_kv_write(const void* k, long k_stride, const void* v, long v_stride, int dtype, int M, int KV, int hd,
                           const int* row_seq, const int* row_pos, const int* new_len, const int* table, int table_w,
                           void* k_pool, void* v_pool, int page, int rows_cap, void* stream) {
    TP_REQUIRE(M > 0 && KV > 0 && hd > 0 && page > 0 && table_w > 0, "kv_write: empty shape");
    TP_REQUIRE(k && v && row_seq && row_pos && new_len && table && k_pool && v_pool, "kv_write: a null operand");
    TP_REQUIRE(k_stride >= (long)KV * hd && v_stride >= (long)KV * hd, "kv_write: rows are too short for %d heads of %d", KV, hd);
    TP_REQUIRE(rows_cap >= 0 && (rows_cap == 0 || rows_cap % page == 0), "kv_write: ring of %d rows is no multiple of the page size %d", rows_cap, page);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TP_BF16)
        kv_write_k<bf16_t><<<M, 256, 0, s>>>((const bf16_t*)k, k_stride, (const bf16_t*)v, v_stride, KV, hd, row_seq, row_pos, new_len,
                                             table, table_w, (bf16_t*)k_pool, (bf16_t*)v_pool, page, rows_cap);
    else if (dtype == TP_F32)
        kv_write_k<float><<<M, 256, 0, s>>>((const float*)k, k_stride, (const float*)v, v_stride, KV, hd, row_seq, row_pos, new_len,
                                            table, table_w, (float*)k_pool, (float*)v_pool, page, rows_cap);
    else return tp_fail("kv_write: unknown dtype %d", dtype);
    return tp_check_launch("kv_write");
}

// ---- gated activation on a packed gate/up product: y [M, 2*Ip] fp32 with 16 gate columns, then the 16 up
// columns of the same units, alternating.  out[m, i] = act(g) * u, act being gelu-tanh (runtime/cuda/codebook_gemv.cu:
// 531-537) or SiLU (the reference's other feed-forward: runtime/cuda/codebook_gemv.cu:205-209), in float32 arithmetic.
// ---- rows += bias: for products with a bias (the products themselves have no bias operand) ------------------------
template <typename T>
__global__ void add_bias_k(T* __restrict__ rows, const float* __restrict__ bias, long total, int N) {
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x)
        st_f32(rows + i, ld_f32(rows + i) + bias[i % N]);
}

extern "C" int tp_add_bias(void* rows, int dtype, const float* bias, int M, int N, void* stream) {
    TP_REQUIRE(rows && bias && M > 0 && N > 0, "add_bias: empty shape M=%d N=%d", M, N);
    const long total = (long)M * N;
    long blocks = (total + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TP_BF16) add_bias_k<bf16_t><<<(unsigned)blocks, 256, 0, s>>>((bf16_t*)rows, bias, total, N);
    else if (dtype == TP_F32) add_bias_k<float><<<(unsigned)blocks, 256, 0, s>>>((float*)rows, bias, total, N);
    else return tp_fail("add_bias: unknown dtype %d", dtype);
    return tp_check_launch("add_bias");
}

template <typename T>
__global__ void gated_act_k(const float* __restrict__ y, T* __restrict__ out, int I, int Ip2, int act) {
    const float* yr = y + (size_t)blockIdx.x * Ip2;
    T* orow = out + (size_t)blockIdx.x * I;
    for (int i = threadIdx.x; i < I; i += blockDim.x) {
        const int base = (i >> 4) * 32 + (i & 15);
        st_f32(orow + i, gate_act_exact(yr[base], act) * yr[base + 16]);
    }
}

extern "C" int tp_gated_act(const float* y, void* out, int dtype, int M, int I, int act, void* stream) {
    TP_REQUIRE(M > 0 && I > 0, "gated_act: empty shape M=%d I=%d", M, I);
    TP_REQUIRE(act == TP_ACT_GELU_TANH || act == TP_ACT_SILU, "gated_act: unknown activation %d", act);
    const int Ip2 = 2 * ((I + 15) / 16) * 16;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TP_BF16) gated_act_k<bf16_t><<<M, 256, 0, s>>>(y, (bf16_t*)out, I, Ip2, act);
    else if (dtype == TP_F32) gated_act_k<float><<<M, 256, 0, s>>>(y, (float*)out, I, Ip2, act);
    else return tp_fail("gated_act: unknown dtype %d", dtype);
    return tp_check_launch("gated_act");
}
