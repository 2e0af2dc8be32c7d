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

// stage 1 of the two-stage form: grid (parts, rows), each block scans one contiguous part of a row
__global__ void __launch_bounds__(256)
argmax_part_k(const float* __restrict__ logits, int V, int per_part, float* __restrict__ pval, int* __restrict__ pidx) {
    __shared__ float sval[4];
    __shared__ int sidx[4];
    const float* z = logits + (size_t)blockIdx.y * V;
    const int lo = blockIdx.x * per_part, hi = min(V, lo + per_part);
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        const float v = z[i];
        if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
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
        for (int w = 1; w < 4; w++)
            if (sval[w] > bv || (sval[w] == bv && sidx[w] < bi)) { bv = sval[w]; bi = sidx[w]; }
        pval[blockIdx.y * gridDim.x + blockIdx.x] = bv;
        pidx[blockIdx.y * gridDim.x + blockIdx.x] = bi;
    }
}

// stage 2: one wave per row over the parts' winners
__global__ void __launch_bounds__(64)
argmax_final_k(const float* __restrict__ pval, const int* __restrict__ pidx, int parts, int* __restrict__ out) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < parts; i += 64) {
        const float v = pval[blockIdx.x * parts + i];
        const int id = pidx[blockIdx.x * parts + i];
        if (v > bv || (v == bv && id < bi)) { bv = v; bi = id; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (threadIdx.x == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
}

extern "C" long tp_argmax_workspace_bytes(int B, int V) {
    const int parts = V >= 16384 ? 64 : 1;
    return parts > 1 ? (long)B * parts * 8 : 0;
}

extern "C" int tp_argmax(const float* logits, int B, int V, int* out, void* workspace, void* stream) {
    TP_REQUIRE(B > 0 && V > 0, "argmax: empty shape B=%d V=%d", B, V);
    TP_REQUIRE(B <= 65535, "argmax: %d rows exceed one launch", B);
    const int parts = V >= 16384 ? 64 : 1;
    hipStream_t s = (hipStream_t)stream;
    if (parts == 1 || !workspace) {
        argmax_k<<<B, 1024, 0, s>>>(logits, V, out);
        return tp_check_launch("argmax");
    }
    float* pval = (float*)workspace;
    int* pidx = (int*)(pval + (size_t)B * parts);
    argmax_part_k<<<dim3(parts, B), 256, 0, s>>>(logits, V, tp_cdiv(V, parts), pval, pidx);
    if (int rc = tp_check_launch("argmax (parts)")) return rc;
    argmax_final_k<<<B, 64, 0, s>>>(pval, pidx, parts, out);
    return tp_check_launch("argmax (final)");
}

// ---- repetition penalty: every distinct recent token once, z / penalty if z > 0 else z * penalty
// (runtime/src/bin/serve.rs:285-294; the reference keeps the last 128 tokens, prompt included, as a set). -----
__global__ void repetition_penalty_k(float* __restrict__ logits, int V, const int* __restrict__ recent, int R, float penalty) {
    float* z = logits + (size_t)blockIdx.x * V;
    const int* rec = recent + (size_t)blockIdx.x * R;
    for (int j = threadIdx.x; j < R; j += blockDim.x) {
        const int t = rec[j];
        if (t < 0 || t >= V) continue;
        bool first = true;
        for (int i = 0; i < j; i++) if (rec[i] == t) { first = false; break; }
        if (!first) continue;
        const float v = z[t];
        z[t] = v > 0.f ? v / penalty : v * penalty;
    }
}

extern "C" int tp_repetition_penalty(float* logits, int B, int V, const int* recent, int R, float penalty, void* stream) {
    TP_REQUIRE(B > 0 && V > 0 && R > 0, "repetition_penalty: empty shape B=%d V=%d R=%d", B, V, R);
    if (penalty <= 1.f) return 0;
    repetition_penalty_k<<<B, 128, 0, (hipStream_t)stream>>>(logits, V, recent, R, penalty);
    return tp_check_launch("repetition_penalty");
}

// ---- temperature sampling over the top_k largest logits with a top_p cut, as the reference's next_tok
// (runtime/src/bin/serve.rs:41-72): candidates sorted by logit descending (ties: smaller id first),
// p = exp((z - max) / T) / sum, the shortest prefix whose cumulative mass reaches top_p, then a walk with
// r = u * kept mass; falls back to the first candidate.  One block per row: a radix select over the value
// bits finds the k-th largest logit, an id select breaks ties at that value, the at most 1024 candidates are
// sorted in LDS, and one thread does the short sequential part in the reference's order of additions. -------
__device__ __forceinline__ uint32_t value_key(float f) {           // larger float -> larger key; NaN lowest
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0u;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
    const uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __uint_as_float(u);
}

__global__ void __launch_bounds__(1024)
sample_k(const float* __restrict__ logits, int V, float temperature, int top_k, float top_p,
         const float* __restrict__ uniforms, int* __restrict__ out) {
    __shared__ unsigned hist[256];
    __shared__ uint32_t ckey[1024];
    __shared__ int cid[1024];
    __shared__ float prob[1024];
    __shared__ unsigned s_prefix, s_remaining, s_count, s_eq_total;
    __shared__ int s_id_limit;
    const float* z = logits + (size_t)blockIdx.x * V;
    const int tid = threadIdx.x;
    const int k = top_k < V ? top_k : V;

    // 1. the k-th largest value key, 8 bits at a time from the top
    if (tid == 0) { s_prefix = 0u; s_remaining = (unsigned)k; }
    for (int shift = 24; shift >= 0; shift -= 8) {
        if (tid < 256) hist[tid] = 0u;
        __syncthreads();
        const unsigned prefix = s_prefix;
        for (int i = tid; i < V; i += blockDim.x) {
            const uint32_t key = value_key(z[i]);
            if (shift == 24 || (key >> (shift + 8)) == (prefix >> (shift + 8))) atomicAdd(&hist[(key >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (tid == 0) {
            unsigned rem = s_remaining;
            int b = 255;
            for (; b > 0; b--) {
                if (hist[b] >= rem) break;
                rem -= hist[b];
            }
            s_prefix = prefix | ((unsigned)b << shift);
            s_remaining = rem;                       // how many of this bucket are still needed
            if (shift == 0) s_eq_total = hist[b];
        }
        __syncthreads();
    }
    const uint32_t tkey = s_prefix;                  // value key of the k-th largest
    const unsigned need_eq = s_remaining;            // candidates to take among those equal to it
    // 2. ties at the threshold: the need_eq smallest ids among the equal ones
    if (tid == 0) s_id_limit = 0x7fffffff;
    __syncthreads();
    if (s_eq_total > need_eq) {
        if (tid == 0) { s_prefix = 0u; s_remaining = need_eq; }
        for (int shift = 24; shift >= 0; shift -= 8) {
            if (tid < 256) hist[tid] = 0u;
            __syncthreads();
            const unsigned prefix = s_prefix;
            for (int i = tid; i < V; i += blockDim.x) {
                if (value_key(z[i]) != tkey) continue;
                const unsigned id = (unsigned)i;
                if (shift == 24 || (id >> (shift + 8)) == (prefix >> (shift + 8))) atomicAdd(&hist[(id >> shift) & 255u], 1u);
            }
            __syncthreads();
            if (tid == 0) {
                unsigned rem = s_remaining;
                int b = 0;
                for (; b < 255; b++) {
                    if (hist[b] >= rem) break;
                    rem -= hist[b];
                }
                s_prefix = prefix | ((unsigned)b << shift);
                s_remaining = rem;
            }
            __syncthreads();
        }
        if (tid == 0) s_id_limit = (int)s_prefix;    // the need_eq-th smallest id among the equal ones
        __syncthreads();
    }
    // 3. collect the k candidates
    if (tid == 0) s_count = 0u;
    ckey[tid] = 0u;
    cid[tid] = 0x7fffffff;
    __syncthreads();
    const int id_limit = s_id_limit;
    for (int i = tid; i < V; i += blockDim.x) {
        const uint32_t key = value_key(z[i]);
        if (key > tkey || (key == tkey && i <= id_limit)) {
            const unsigned at = atomicAdd(&s_count, 1u);
            if (at < 1024u) { ckey[at] = key; cid[at] = i; }
        }
    }
    __syncthreads();
    // 4. sort the 1024 entries by (key descending, id ascending); empty entries (key 0, id max) sink
    for (int size = 2; size <= 1024; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            const int partner = tid ^ stride;
            if (partner > tid) {
                const bool descending = (tid & size) == 0;
                const uint32_t ka = ckey[tid], kb = ckey[partner];
                const int ia = cid[tid], ib = cid[partner];
                const bool a_first = ka > kb || (ka == kb && ia < ib);      // a belongs before b
                if (a_first != descending) { ckey[tid] = kb; ckey[partner] = ka; cid[tid] = ib; cid[partner] = ia; }
            }
            __syncthreads();
        }
    }
    // 5. probabilities, the nucleus and the draw
    const float mx = key_value(ckey[0]);
    if (tid < k) prob[tid] = expf((key_value(ckey[tid]) - mx) / temperature);
    __syncthreads();
    if (tid == 0) {
        float sum = 0.f;
        for (int j = 0; j < k; j++) sum += prob[j];
        for (int j = 0; j < k; j++) prob[j] /= sum;
        float cum = 0.f;
        int keep = k;
        for (int j = 0; j < k; j++) {
            cum += prob[j];
            if (cum >= top_p) { keep = j + 1; break; }
        }
        float kept = 0.f;
        for (int j = 0; j < keep; j++) kept += prob[j];
        float r = uniforms[blockIdx.x] * kept;
        int pick = cid[0];
        for (int j = 0; j < keep; j++) {
            if (r < prob[j]) { pick = cid[j]; break; }
            r -= prob[j];
        }
        out[blockIdx.x] = pick;
    }
}

extern "C" int tp_sample(const float* logits, int B, int V, float temperature, int top_k, float top_p,
                         const float* uniforms, int* out, void* stream) {
    TP_REQUIRE(B > 0 && V > 0, "sample: empty shape B=%d V=%d", B, V);
    TP_REQUIRE(temperature > 0.f, "sample: temperature %g must be positive (0 means argmax)", temperature);
    TP_REQUIRE(top_k >= 1 && top_k <= 1024, "sample: top_k %d must lie in 1..1024", top_k);
    TP_REQUIRE(top_p > 0.f, "sample: top_p %g must be positive", top_p);
    sample_k<<<B, 1024, 0, (hipStream_t)stream>>>(logits, V, temperature, top_k, top_p, uniforms, out);
    return tp_check_launch("sample");
}
