// Token choice on the device: argmax, repetition penalty, temperature / top-k / top-p sampling.
#include "common.h"
#include "no_alloc.h"
#include <mutex>

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

// ---- argmax for callers that cannot allocate (declared in no_alloc.h) -------------------------------------------
// The two-stage form above with the parts' winners in a file-scope device array instead of a caller's workspace.
// Every GPU the library runs on holds its own copy of the array (128 KiB) until the process ends; in host code the
// array's name is only a handle, so its device address is asked for once per device (hipGetSymbolAddress with that
// device current) and kept.  Nothing in the array has to start at zero: stage 2 reads exactly the B * parts pairs
// that stage 1 of the same call wrote.  All calls on one GPU share the array: calls that overlap there (two
// streams, two threads) race.
static __device__ __align__(256) unsigned char scratch[TP_ARGMAX_NO_ALLOC_SCRATCH_BYTES];

namespace {
constexpr int NO_ALLOC_MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[NO_ALLOC_MAX_DEVICES];        // per device: where that GPU's copy of `scratch` lies

int scratch_address(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return tp_fail("argmax_no_alloc: no current device: %s", hipGetErrorString(e));
    TP_REQUIRE(dev >= 0 && dev < NO_ALLOC_MAX_DEVICES, "argmax_no_alloc: device %d is beyond the %d this library keeps track of", dev, NO_ALLOC_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return tp_fail("argmax_no_alloc: the scratch array's address on device %d is not available: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}
}  // namespace

extern "C" int tp_argmax_no_alloc_prepare(void) {
    void* base = nullptr;
    return scratch_address(&base);
}

extern "C" int tp_argmax_no_alloc(const float* logits, int B, int V, int* out, void* stream) {
    TP_REQUIRE(logits && out, "argmax_no_alloc: logits and output must be given");
    TP_REQUIRE(B > 0 && V > 0, "argmax_no_alloc: empty shape B=%d V=%d", B, V);
    TP_REQUIRE(B <= TP_ARGMAX_NO_ALLOC_MAX_ROWS, "argmax_no_alloc: %d rows exceed the %d that the fixed scratch array holds",
               B, TP_ARGMAX_NO_ALLOC_MAX_ROWS);
    static_assert((size_t)TP_ARGMAX_NO_ALLOC_MAX_ROWS * TP_ARGMAX_NO_ALLOC_PARTS * 8 <= TP_ARGMAX_NO_ALLOC_SCRATCH_BYTES,
                  "the scratch array must hold a (value, index) pair per row and part");
    void* base = nullptr;
    if (int rc = scratch_address(&base)) return rc;
    const int parts = TP_ARGMAX_NO_ALLOC_PARTS;
    float* pval = (float*)base;
    int* pidx = (int*)(pval + (size_t)B * parts);
    hipStream_t s = (hipStream_t)stream;
    argmax_part_k<<<dim3(parts, B), 256, 0, s>>>(logits, V, tp_cdiv(V, parts), pval, pidx);
    if (int rc = tp_check_launch("argmax_no_alloc (parts)")) return rc;
    argmax_final_k<<<B, 64, 0, s>>>(pval, pidx, parts, out);
    return tp_check_launch("argmax_no_alloc (final)");
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

// The recent tokens of a row as a ring on the device, so that a captured decode graph can keep them by itself: the
// row's chosen id goes to the place its cursor names, and the cursor moves on (the oldest id is overwritten once
// the ring is full; the penalty reads the ring as a set, so the order inside it does not matter).
__global__ void recent_push_k(const int* __restrict__ tokens, int* __restrict__ recent, int* __restrict__ cursor, int B, int R) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= B) return;
    int at = cursor[i];
    at = at < 0 || at >= R ? 0 : at;
    recent[(size_t)i * R + at] = tokens[i];
    cursor[i] = at + 1 == R ? 0 : at + 1;
}

extern "C" int tp_recent_push(const int* tokens, int* recent, int* cursor, int B, int R, void* stream) {
    TP_REQUIRE(tokens && recent && cursor && B > 0 && R > 0, "recent_push: empty shape B=%d R=%d", B, R);
    recent_push_k<<<tp_cdiv(B, 64), 64, 0, (hipStream_t)stream>>>(tokens, recent, cursor, B, R);
    return tp_check_launch("recent_push");
}

// ---- temperature sampling over the top_k largest logits with a top_p cut, as the reference's next_tok
// (runtime/src/bin/serve.rs:41-72): candidates sorted by logit descending (ties: smaller id first),
// p = exp((z - max) / T) / sum, the shortest prefix whose cumulative mass reaches top_p, then a walk with
// r = u * kept mass; falls back to the first candidate.  One block per row: a radix select over the value
// bits finds the k-th largest logit, an id select breaks ties at that value, the at most 1024 candidates are
// sorted in LDS, and the first wave does the short scans (sums in candidate order within a lane, then over the lanes). ---
__device__ __forceinline__ uint32_t value_key(float f) {           // larger float -> larger key; NaN lowest
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0u;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
    const uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __uint_as_float(u);
}

// ---- the sampler's short scans, done by the block's first wave (a single thread walking LDS pays its latency per
// element: 45 us for 256 candidates) -----------------------------------------------------------------------------
__device__ __forceinline__ unsigned wave_scan_incl(unsigned v, int lane) {
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const unsigned t = (unsigned)__shfl_up((int)v, o, 64);
        if (lane >= o) v += t;
    }
    return v;
}
__device__ __forceinline__ float wave_scan_incl(float v, int lane) {
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float t = __shfl_up(v, o, 64);
        if (lane >= o) v += t;
    }
    return v;
}
// Walks the 256 counters from the top (or from the bottom) until `rem` of them are covered: the bucket that holds the
// rem-th member, and how many of that bucket are still needed.  All 64 lanes of one wave call it.
__device__ __forceinline__ void pick_bucket(const unsigned* hist, bool from_top, unsigned rem, int lane, int& bucket, unsigned& rem_out) {
    unsigned c[4], local = 0u;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int o = lane * 4 + j;
        c[j] = hist[from_top ? 255 - o : o];
        local += c[j];
    }
    const unsigned incl = wave_scan_incl(local, lane);
    const unsigned long long hit = __ballot(incl >= rem);
    const int L = hit ? __ffsll((long long)hit) - 1 : 63;
    unsigned r = rem - (incl - local);
    int j = 0;
    for (; j < 3; j++) {
        if (c[j] >= r) break;
        r -= c[j];
    }
    const int o = L * 4 + __shfl(j, L, 64);
    bucket = from_top ? 255 - o : o;
    rem_out = (unsigned)__shfl((int)r, L, 64);
}

// With a candidate list (cand_count non-null): row b's candidates are cand_val/cand_id[b * cand_cap ..], a superset
// of its top_k if their number fits cand_cap; the kernel then works on the list, else on the whole row.
__global__ void __launch_bounds__(1024)
sample_k(const float* __restrict__ logits, int V, float temperature, int top_k, float top_p,
         const float* __restrict__ uniforms, int* __restrict__ out,
         const unsigned* __restrict__ cand_count, const float* __restrict__ cand_val, const int* __restrict__ cand_id,
         int cand_cap) {
    __shared__ unsigned hist[256];
    __shared__ uint32_t ckey[1024];
    __shared__ int cid[1024];
    __shared__ float prob[1024];
    __shared__ unsigned s_prefix, s_remaining, s_count, s_eq_total;
    __shared__ int s_id_limit;
    const float* z = logits + (size_t)blockIdx.x * V;
    const int tid = threadIdx.x;
    const int k = top_k < V ? top_k : V;                       // of the whole row, whichever source is read
    const int* ids = nullptr;                                  // candidate -> token id; null: the index is the id
    if (cand_count && cand_count[blockIdx.x] <= (unsigned)cand_cap && cand_count[blockIdx.x] >= (unsigned)k) {
        V = (int)cand_count[blockIdx.x];
        z = cand_val + (size_t)blockIdx.x * cand_cap;
        ids = cand_id + (size_t)blockIdx.x * cand_cap;
    }

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
        if (tid < 64) {
            int b;
            unsigned rem;
            pick_bucket(hist, true, s_remaining, tid, b, rem);
            if (tid == 0) {
                s_prefix = prefix | ((unsigned)b << shift);
                s_remaining = rem;                   // how many of this bucket are still needed
                if (shift == 0) s_eq_total = hist[b];
            }
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
                const unsigned id = (unsigned)(ids ? ids[i] : i);
                if (shift == 24 || (id >> (shift + 8)) == (prefix >> (shift + 8))) atomicAdd(&hist[(id >> shift) & 255u], 1u);
            }
            __syncthreads();
            if (tid < 64) {
                int b;
                unsigned rem;
                pick_bucket(hist, false, s_remaining, tid, b, rem);
                if (tid == 0) {
                    s_prefix = prefix | ((unsigned)b << shift);
                    s_remaining = rem;
                }
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
        const int id = ids ? ids[i] : i;
        if (key > tkey || (key == tkey && id <= id_limit)) {
            const unsigned at = atomicAdd(&s_count, 1u);
            if (at < 1024u) { ckey[at] = key; cid[at] = id; }
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
    // 5. probabilities, the nucleus and the draw: the first wave, each lane 16 consecutive candidates; sums run over a
    // lane's candidates in order, then over the lanes in order
    const float mx = key_value(ckey[0]);
    if (tid < k) prob[tid] = expf((key_value(ckey[tid]) - mx) / temperature);
    __syncthreads();
    if (tid < 64) {
        const int j0 = tid * 16;
        float local = 0.f;
        for (int j = j0; j < j0 + 16 && j < k; j++) local += prob[j];
        const float total = __shfl(wave_scan_incl(local, tid), 63, 64);
        // cumulative probabilities (reusing the key array's space: 1024 floats)
        float* cum = reinterpret_cast<float*>(ckey);
        float lsum = 0.f;
        for (int j = j0; j < j0 + 16 && j < k; j++) { prob[j] /= total; lsum += prob[j]; }
        float run = wave_scan_incl(lsum, tid) - lsum;
        for (int j = j0; j < j0 + 16 && j < k; j++) { run += prob[j]; cum[j] = run; }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // the shortest prefix whose mass reaches top_p
        int first = k;
        for (int j = j0; j < j0 + 16 && j < k; j++)
            if (cum[j] >= top_p) { first = j; break; }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) first = min(first, __shfl_xor(first, o, 64));
        const int keep = first < k ? first + 1 : k;
        const float kept = cum[keep - 1];
        const float r = uniforms[blockIdx.x] * kept;
        // the walk: the first candidate whose cumulative mass exceeds r; none (rounding at the end): the first candidate
        int hit = keep;
        for (int j = j0; j < j0 + 16 && j < keep; j++)
            if (r < cum[j]) { hit = j; break; }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) hit = min(hit, __shfl_xor(hit, o, 64));
        if (tid == 0) out[blockIdx.x] = cid[hit < keep ? hit : 0];
    }
}

// ---- temperature sampling over the whole vocabulary (top_k 0, no nucleus; the reference always keeps 256): p_i =
// exp((z_i - max) / T), r = u * sum, the token whose cumulative mass in id order first exceeds r.  One block per
// row; thread t owns a contiguous range of ids, so sums run over ids in order within a thread, then over the threads
// in order. ----------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(1024)
sample_full_k(const float* __restrict__ logits, int V, float temperature, const float* __restrict__ uniforms,
              int* __restrict__ out) {
    __shared__ float part[1024];
    __shared__ float s_total;
    __shared__ int s_winner;
    const float* z = logits + (size_t)blockIdx.x * V;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float mx = -INFINITY;
    for (int i = tid; i < V; i += 1024) { const float v = z[i]; mx = v > mx ? v : mx; }      // NaN never wins
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    if (lane == 0) part[wave] = mx;
    __syncthreads();
    mx = part[0];
    for (int w = 1; w < 16; w++) mx = fmaxf(mx, part[w]);
    __syncthreads();
    const int chunk = (V + 1023) / 1024, begin = tid * chunk, end = min(V, begin + chunk);
    float mine = 0.f;
    for (int i = begin; i < end; i++) { const float v = z[i]; mine += v == v ? expf((v - mx) / temperature) : 0.f; }
    part[tid] = mine;
    __syncthreads();
    if (tid < 64) {                                  // the first wave: totals of 16 threads per lane, then over the lanes
        float local = 0.f;
        for (int j = 0; j < 16; j++) local += part[tid * 16 + j];
        const float incl = wave_scan_incl(local, tid);
        float run = incl - local;
        for (int j = 0; j < 16; j++) { const float v = part[tid * 16 + j]; part[tid * 16 + j] = run; run += v; }   // exclusive sums
        if (tid == 63) s_total = incl;
    }
    __syncthreads();
    const float r = uniforms[blockIdx.x] * s_total;
    const float before = part[tid];
    // the first thread whose range reaches past r walks it; rounding may leave r past every range: the last one
    if (tid == 0) s_winner = (V - 1) / chunk;
    __syncthreads();
    if (begin < end && r < before + mine) atomicMin(&s_winner, tid);
    __syncthreads();
    if (tid == s_winner) {
        float run = before;
        int pick = end - 1;
        for (int i = begin; i < end; i++) {
            const float v = z[i];
            run += v == v ? expf((v - mx) / temperature) : 0.f;
            if (r < run) { pick = i; break; }
        }
        out[blockIdx.x] = pick;
    }
}

// ---- a coarse filter in front of the exact sampler, on many blocks: the sampler alone reads a row of 256,000
// logits several times on one CU (0.4 ms).  A histogram of the top 12 bits of the value keys gives the bin that
// holds the top_k-th largest logit; everything from that bin upwards (top_k plus that bin's other members, a few
// hundred for logits of a language model) is copied to a candidate list, which the sampler then works on.  A list
// that would not fit falls back to the whole row, so the result never depends on the filter. -------------------
constexpr int FILTER_BINS = 4096;
constexpr int FILTER_PART = 8192;                    // logits per block

__global__ void __launch_bounds__(256)
filter_hist_k(const float* __restrict__ logits, int V, unsigned* __restrict__ hist) {
    __shared__ unsigned local[FILTER_BINS];
    for (int i = threadIdx.x; i < FILTER_BINS; i += 256) local[i] = 0u;
    __syncthreads();
    const float* z = logits + (size_t)blockIdx.y * V;
    const int begin = blockIdx.x * FILTER_PART, end = min(V, begin + FILTER_PART);
    for (int i = begin + threadIdx.x; i < end; i += 256) atomicAdd(&local[value_key(z[i]) >> 20], 1u);
    __syncthreads();
    unsigned* row = hist + (size_t)blockIdx.y * FILTER_BINS;
    for (int i = threadIdx.x; i < FILTER_BINS; i += 256)
        if (local[i]) atomicAdd(&row[i], local[i]);
}

// the bin of the k-th largest key; the histogram and the candidate counter are left zeroed for the next call
__global__ void __launch_bounds__(256)
filter_bin_k(unsigned* __restrict__ hist, int k, unsigned* __restrict__ bin_out, unsigned* __restrict__ cand_count) {
    __shared__ unsigned part[256];
    unsigned* row = hist + (size_t)blockIdx.x * FILTER_BINS;
    const int tid = threadIdx.x;
    constexpr int PER = FILTER_BINS / 256;           // thread t owns bins t*PER .. t*PER+PER-1
    unsigned mine[PER], sum = 0u;
#pragma unroll
    for (int j = 0; j < PER; j++) { mine[j] = row[tid * PER + j]; sum += mine[j]; row[tid * PER + j] = 0u; }
    part[tid] = sum;
    __syncthreads();
    if (tid == 0) {
        unsigned above = 0u;                         // members of the bins above the current thread's
        int t = 255;
        for (; t > 0; t--) {
            if (above + part[t] >= (unsigned)k) break;
            above += part[t];
        }
        part[0] = (unsigned)t;
        part[1] = above;
        cand_count[blockIdx.x] = 0u;
    }
    __syncthreads();
    if (tid == (int)part[0]) {
        unsigned above = part[1];
        int j = PER - 1;
        for (; j > 0; j--) {
            if (above + mine[j] >= (unsigned)k) break;
            above += mine[j];
        }
        bin_out[blockIdx.x] = (unsigned)(tid * PER + j);
    }
}

// a block gathers its candidates in LDS and reserves their places with one addition to the row's counter
__global__ void __launch_bounds__(256)
filter_collect_k(const float* __restrict__ logits, int V, const unsigned* __restrict__ bin, unsigned* __restrict__ cand_count,
                 float* __restrict__ cand_val, int* __restrict__ cand_id, int cand_cap) {
    constexpr int LOCAL = 1024;
    __shared__ float lval[LOCAL];
    __shared__ int lid[LOCAL];
    __shared__ unsigned lcount, base;
    if (threadIdx.x == 0) lcount = 0u;
    __syncthreads();
    const float* z = logits + (size_t)blockIdx.y * V;
    const unsigned lowest = bin[blockIdx.y];
    const int begin = blockIdx.x * FILTER_PART, end = min(V, begin + FILTER_PART);
    for (int i = begin + threadIdx.x; i < end; i += 256) {
        const float v = z[i];
        if ((value_key(v) >> 20) >= lowest) {
            const unsigned at = atomicAdd(&lcount, 1u);
            if (at < (unsigned)LOCAL) { lval[at] = v; lid[at] = i; }
        }
    }
    __syncthreads();
    const unsigned n = lcount;
    if (n == 0u) return;
    // more than the block can hold: the row's count is pushed past the capacity, and the sampler reads the whole row
    if (threadIdx.x == 0) base = atomicAdd(&cand_count[blockIdx.y], n <= (unsigned)LOCAL ? n : (unsigned)cand_cap + 1u);
    __syncthreads();
    if (n > (unsigned)LOCAL) return;
    for (unsigned j = threadIdx.x; j < n; j += 256) {
        const unsigned at = base + j;
        if (at < (unsigned)cand_cap) {
            cand_val[(size_t)blockIdx.y * cand_cap + at] = lval[j];
            cand_id[(size_t)blockIdx.y * cand_cap + at] = lid[j];
        }
    }
}

constexpr int CAND_CAP = 8192;

// bytes of the sampler's workspace for B rows; it must be zero before its first use and is left ready for the next
extern "C" long tp_sample_workspace_bytes(int B, int V) {
    if (V < 4 * FILTER_PART) return 0;               // small vocabularies: the sampler alone
    return (long)B * (FILTER_BINS * 4 + 8 + (long)CAND_CAP * 8);
}

extern "C" int tp_sample(const float* logits, int B, int V, float temperature, int top_k, float top_p,
                         const float* uniforms, int* out, void* workspace, void* stream) {
    TP_REQUIRE(B > 0 && V > 0, "sample: empty shape B=%d V=%d", B, V);
    TP_REQUIRE(temperature > 0.f, "sample: temperature %g must be positive (0 means argmax)", temperature);
    TP_REQUIRE(top_k >= 0 && top_k <= 1024, "sample: top_k %d must lie in 0..1024 (0: the whole vocabulary)", top_k);
    TP_REQUIRE(top_p > 0.f, "sample: top_p %g must be positive", top_p);
    TP_REQUIRE(top_k > 0 || top_p >= 1.f, "sample: a nucleus (top_p %g) needs top_k between 1 and 1024", top_p);
    TP_REQUIRE(B <= 65535, "sample: %d rows exceed one launch", B);
    hipStream_t s = (hipStream_t)stream;
    if (top_k == 0) {
        sample_full_k<<<B, 1024, 0, s>>>(logits, V, temperature, uniforms, out);
        return tp_check_launch("sample (whole vocabulary)");
    }
    if (!workspace || tp_sample_workspace_bytes(B, V) == 0) {
        sample_k<<<B, 1024, 0, s>>>(logits, V, temperature, top_k, top_p, uniforms, out, nullptr, nullptr, nullptr, 0);
        return tp_check_launch("sample");
    }
    unsigned* hist = (unsigned*)workspace;
    unsigned* bin = hist + (size_t)B * FILTER_BINS;
    unsigned* count = bin + B;
    float* cand_val = (float*)(count + B);
    int* cand_id = (int*)(cand_val + (size_t)B * CAND_CAP);
    const dim3 grid(tp_cdiv(V, FILTER_PART), B);
    filter_hist_k<<<grid, 256, 0, s>>>(logits, V, hist);
    if (int rc = tp_check_launch("sample (histogram)")) return rc;
    filter_bin_k<<<B, 256, 0, s>>>(hist, top_k < V ? top_k : V, bin, count);
    if (int rc = tp_check_launch("sample (threshold bin)")) return rc;
    filter_collect_k<<<grid, 256, 0, s>>>(logits, V, bin, count, cand_val, cand_id, CAND_CAP);
    if (int rc = tp_check_launch("sample (candidates)")) return rc;
    sample_k<<<B, 1024, 0, s>>>(logits, V, temperature, top_k, top_p, uniforms, out, count, cand_val, cand_id, CAND_CAP);
    return tp_check_launch("sample");
}
