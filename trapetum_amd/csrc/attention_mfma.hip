// bf16 attention of decode steps on the matrix cores for one head size (compiled with -DTP_HD=<head_dim>, a
// multiple of 16 up to 256): one query per sequence and head over the paged cache.  (Steps of many queries:
// attention_prefill.hip, in the same library.)
//
// Formula as the reference's attn_k (runtime/cuda/codebook_gemv.cu:240-270): score = (q . k) * scale, then
// cap * tanh(score / cap) if a cap is set, softmax over the visible keys in fp32, weighted sum of v, query head
// h reading kv head h / (heads / kv_heads).  The scale is an argument (rsqrt(head_dim) in the reference), and a
// window W hides keys with p - t >= W (the reference has none: runtime/src/lib.rs:4455).
//
// Scores are computed transposed, S^T = K . Q^T with v_mfma_f32_16x16x32_bf16: key rows are the A operand (a
// lane holds 8 consecutive elements of one key: one 16-byte load), queries the B operand, and a lane ends up
// with 4 keys of ONE query, so the softmax statistics are per-lane scalars.
#include "common.h"
#include <type_traits>
#include "error_channel.h"

#ifndef TP_HD
#error "compile with -DTP_HD=<head_dim>"
#endif

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

namespace {
constexpr int HD = TP_HD;
constexpr int HDP = (HD + 31) / 32 * 32;       // head size padded to the product's k step
constexpr int KSTEPS = HDP / 32;
constexpr int NCH = HD / 8;                     // 16-byte chunks of a row
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head_dim must be a multiple of 16 up to 256");

union Frag { uint4 u; bf16x8 v; bf16_t h[8]; };

__device__ __forceinline__ bf16x8 ld_frag(const bf16_t* p, bool ok) {
    Frag f;
    if (ok) f.u = *reinterpret_cast<const uint4*>(p);
    else f.u = make_uint4(0, 0, 0, 0);
    return f.v;
}
// tanh through one exponential and one reciprocal: 1 - 2 / (1 + e^(2x)); exact at both ends, relative error of a
// few 1e-7 elsewhere (the scores are rounded to bf16 probabilities afterwards)
__device__ __forceinline__ float tanh_fast(float x) {
    return 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __expf(2.f * x));
}
// scale_over_cap = scale / cap, so that a capped score costs two multiplications around the tanh
__device__ __forceinline__ float score_of(float dot, float scale, float cap, float scale_over_cap) {
    return cap > 0.f ? cap * tanh_fast(dot * scale_over_cap) : dot * scale;
}
__device__ __forceinline__ bf16_t bf16_bits(float f) {
    __bf16 b = (__bf16)f;                          // one conversion instruction on gfx950, round to nearest even
    return __builtin_bit_cast(bf16_t, b);
}
}  // namespace

// =====================================================================================================
// decode: one query per sequence and head, keys and values in the paged cache.  A block owns one
// (sequence, kv head, slice of the keys) and all the query heads of that kv head, so K and V are read once
// for the group.  Scores by MFMA with key rows loaded straight from global memory; probabilities through
// a wave's LDS; the weighted sum of V with plain FMAs (V's rows are contiguous along the head, not along the
// keys), each lane owning one 16-byte chunk of the head for a subset of the wave's 16 keys.  A wave keeps its
// own running softmax over the keys it sees, so the waves of a block meet only once, at the end; a round's value
// chunks are fetched together with its key rows, before the scores are known, so the two latencies overlap.  Slices of the keys
// (flash-decoding) write (max, sum, unnormalised output) to a workspace that a second kernel combines in
// slice order.
// =====================================================================================================
struct DecodeArgs {
    const bf16_t* q; long q_stride; int H, KV; const int* new_len; const int* table; int table_w;
    bf16_t* k_pool; bf16_t* v_pool; int page, rows_cap; float scale, cap; int window;
    bf16_t* out; float* ws_o; float* ws_ml; int nsplit;
    // the step's projections, when the kernel rotates and caches them itself (else null): rows of
    // [heads | kv heads (keys) | kv heads (values)] x head size, bf16, or float32 in K slices that are added here
    const void* qkv; int qkv_f32, n_slices; long slice_stride, row_stride;
    const float* inv_freq; int rot, write_kv;
};

namespace {
// In the decode kernel a lane's two loads of a pair of product steps are adjacent 16-byte pieces, so the four lanes
// of a key row fetch a whole 128-byte line per pair: step ks, lane group g -> head elements dofs .. dofs + 7.
constexpr int DSTEPS = 2 * ((HD + 63) / 64);
__device__ __forceinline__ int dofs(int ks, int g) { return (ks >> 1) * 64 + g * 16 + (ks & 1) * 8; }
constexpr int DTH = 256;                         // 4 waves; each scores and sums its own 16 keys of a round
constexpr int ROUND = 64;                        // keys a block takes per round
constexpr int KGW = 64 / NCH > 16 ? 16 : 64 / NCH;   // key groups of a wave: lanes with one chunk index walk the keys KGW apart
constexpr int VPT = (16 + KGW - 1) / KGW;        // value chunks a lane fetches per round
}

template <int QT>
__global__ void __launch_bounds__(DTH)
attn_decode_k(DecodeArgs a) {
    __shared__ float p_lds[4][QT][16];               // a wave's probabilities of its 16 keys
    __shared__ float alpha_lds[4][QT];
    __shared__ float m_w[4][QT], l_w[4][QT];
    __shared__ float red[4 * KGW * HD];
    __shared__ __attribute__((aligned(16))) bf16_t q_lds[QT * HD];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 15, g = lane >> 4;
    const int kvh = blockIdx.x, seq = blockIdx.y, split = blockIdx.z;
    const int G = a.H / a.KV;
    const int p = a.new_len[seq] - 1;
    const int lo = a.window > 0 ? max(0, p - a.window + 1) : 0;
    const int lo_al = lo & ~15;
    int chunk = (p + 1 - lo_al + a.nsplit - 1) / a.nsplit;
    chunk = (chunk + ROUND - 1) / ROUND * ROUND;
    const int t_begin = lo_al + split * chunk;
    const int t_end = min(p + 1, t_begin + chunk);
    if (t_begin > p) {                               // this slice has no keys (only when there are several)
        if (tid < G) {
            float* ml = a.ws_ml + (((size_t)seq * a.H + kvh * G + tid) * a.nsplit + split) * 2;
            ml[0] = -INFINITY;
            ml[1] = 0.f;
        }
        return;
    }
    const int* table = a.table + (size_t)seq * a.table_w;
    // Where the 16 keys of a tile live.  Tiles start at multiples of 16 positions; position t is row t, or row
    // t % rows_cap of a ring (rows_cap a multiple of the page size, the page size a power of two >= 16), so a tile
    // lies in one page, in 16 consecutive rows: one page-table entry per tile, looked up once for the wave.
    const int page_shift = __ffs(a.page) - 1, page_mask = a.page - 1;
    const int ring_lo = a.rows_cap > 0 ? lo_al % a.rows_cap : 0;
    auto tile_offset = [&](int tb) -> size_t {                     // element offset of the tile's first row in a pool
        int row = tb;
        if (a.rows_cap > 0) {
            row = ring_lo + (tb - lo_al);
            row = row >= a.rows_cap ? row - a.rows_cap : row;
        }
        const int pg = table[row >> page_shift];
        return (((size_t)pg * a.KV + kvh) * a.page + (row & page_mask)) * HD;
    };

    // the lane's part in the weighted sum: chunk ch of the head, keys kgw, kgw + KGW, ... of the wave's 16
    const int ch = lane % NCH, kgw = lane / NCH;
    const bool pv_lane = kgw < KGW;
    // ---- loads of a round: the key row of lane c for the scores, value chunks for the sum.  Unconditional loads of
    // rows that exist: a hidden or surplus key gets probability 0 (or is skipped) in the sum ---------------------
    auto load_round = [&](int tb, bf16x8 (&kf)[DSTEPS], Frag (&vf)[VPT]) {
        const size_t tile = tile_offset(__builtin_amdgcn_readfirstlane(tb));
        int tk = tb + c;
        tk = tk < lo ? lo : (tk > p ? p : tk);
        const bf16_t* kp = a.k_pool + tile + (size_t)(tk - tb) * HD;
#pragma unroll
        for (int ks = 0; ks < DSTEPS; ks++) {
            const int d0 = dofs(ks, g);
            kf[ks] = ld_frag(kp + (d0 < HD ? d0 : 0), d0 < HD);
        }
#pragma unroll
        for (int j = 0; j < VPT; j++) {
            int kk = kgw + j * KGW;
            kk = kk > 15 ? 15 : kk;
            int tv = tb + kk;
            tv = tv < lo ? lo : (tv > p ? p : tv);
            vf[j].u = *reinterpret_cast<const uint4*>(a.v_pool + tile + (size_t)(tv - tb) * HD + ch * 8);
        }
    };
    // The wave's first round is fetched while the queries are prepared, unless its tile holds the row that this
    // block is about to write.
    bf16x8 kf[DSTEPS];
    Frag vf[VPT];
    const int tb0 = t_begin + wave * 16;
    const bool late = a.qkv && a.write_kv && tb0 <= p && p < tb0 + 16;
    if (tb0 < t_end && !late) load_round(tb0, kf, vf);

    // ---- the group's queries into LDS; in the fused form from the step's projections: K slices added, queries and
    // the new key rotated (pair (f, f + rot/2), angle p * inv_freq[f], in float32), and the slice that holds position
    // p writes the key and the value into the cache before anyone in the block reads that row ---------------------
    if (a.qkv) {
        const int half = a.rot >> 1, rest = HD - a.rot;
        // NC columns of the sequence's row at once: their loads are asked for together (of float32 slices four slices
        // at a time, added in slice order), so that a thread pays one trip to memory for all it needs, not one a column
        auto vals = [&](auto ncol, const long* cols, float* out) {
            constexpr int NC = decltype(ncol)::value;
            if (a.qkv_f32) {
                const float* src = (const float*)a.qkv + (size_t)seq * a.row_stride;
#pragma unroll
                for (int c = 0; c < NC; c++) out[c] = 0.f;
                for (int s0 = 0; s0 < a.n_slices; s0 += 4) {
                    float part[NC][4];
#pragma unroll
                    for (int c = 0; c < NC; c++)
#pragma unroll
                        for (int u = 0; u < 4; u++)
                            part[c][u] = src[(size_t)(s0 + u < a.n_slices ? s0 + u : a.n_slices - 1) * a.slice_stride + cols[c]];
#pragma unroll
                    for (int c = 0; c < NC; c++)
#pragma unroll
                        for (int u = 0; u < 4; u++) out[c] += s0 + u < a.n_slices ? part[c][u] : 0.f;
                }
            } else {
                const bf16_t* src = (const bf16_t*)a.qkv + (size_t)seq * a.row_stride;
#pragma unroll
                for (int c = 0; c < NC; c++) out[c] = bf16_to_f32(src[cols[c]]);
            }
        };
        // the slice that holds position p (t_begin <= p holds here) also rotates the new key and writes it and the value
        // into the cache: thread f < rot/2 does that beside its pair of the first query head, whose angle is the same
        const bool writer = a.write_kv && p < t_begin + chunk;
        bf16_t* kdst = nullptr;
        bf16_t* vdst = nullptr;
        if (writer) {
            int row = a.rows_cap > 0 ? p % a.rows_cap : p;
            const int pg = table[row >> page_shift];
            const size_t at = (((size_t)pg * a.KV + kvh) * a.page + (row & page_mask)) * HD;
            kdst = a.k_pool + at;
            vdst = a.v_pool + at;
        }
        const long kcol = (long)(a.H + kvh) * HD, vcol = (long)(a.H + a.KV + kvh) * HD;
        for (int idx = tid; idx < G * half; idx += DTH) {
            const int qi = idx / half, f = idx - qi * half;
            const long col = (long)(kvh * G + qi) * HD;
            const bool kv = writer && idx < half;                 // then qi == 0 and f == idx
            const long cols[6] = {col + f, col + f + half, kcol + f, kcol + f + half, vcol + f, vcol + f + half};
            float x[6];
            if (writer) vals(std::integral_constant<int, 6>(), cols, x);     // (the whole block takes this branch or the other)
            else vals(std::integral_constant<int, 2>(), cols, x);
            const float ang = (float)p * a.inv_freq[f];
            float cs, sn;
            sincosf(ang, &sn, &cs);
            q_lds[qi * HD + f] = f32_to_bf16(x[0] * cs - x[1] * sn);
            q_lds[qi * HD + f + half] = f32_to_bf16(x[1] * cs + x[0] * sn);
            if (kv) {
                kdst[f] = f32_to_bf16(x[2] * cs - x[3] * sn);
                kdst[f + half] = f32_to_bf16(x[3] * cs + x[2] * sn);
                vdst[f] = f32_to_bf16(x[4]);
                vdst[f + half] = f32_to_bf16(x[5]);
            }
        }
        for (int idx = tid; idx < G * rest; idx += DTH) {         // elements outside the rotation
            const int qi = idx / rest, d = a.rot + idx - qi * rest;
            const bool kv = writer && idx < rest;                 // then qi == 0
            const long cols[3] = {(long)(kvh * G + qi) * HD + d, kcol + d, vcol + d};
            float x[3];
            if (writer) vals(std::integral_constant<int, 3>(), cols, x);
            else vals(std::integral_constant<int, 1>(), cols, x);
            q_lds[qi * HD + d] = f32_to_bf16(x[0]);
            if (kv) {
                kdst[d] = f32_to_bf16(x[1]);
                vdst[d] = f32_to_bf16(x[2]);
            }
        }
        if (writer) __threadfence_block();
    } else {
        for (int idx = tid; idx < G * HD; idx += DTH)
            q_lds[idx] = a.q[(size_t)seq * a.q_stride + (size_t)kvh * G * HD + idx];
    }
    __syncthreads();
    bf16x8 qf[DSTEPS];
#pragma unroll
    for (int ks = 0; ks < DSTEPS; ks++) {
        const int d0 = dofs(ks, g);
        const bool ok = c < G && d0 < HD;
        Frag f;
        f.u = *reinterpret_cast<const uint4*>(q_lds + (ok ? c * HD + d0 : 0));
        const uint32_t keep = (uint32_t) - (int)ok;
        f.u.x &= keep; f.u.y &= keep; f.u.z &= keep; f.u.w &= keep;
        qf[ks] = f.v;
    }
    float acc[QT][8];
#pragma unroll
    for (int qi = 0; qi < QT; qi++)
#pragma unroll
        for (int e = 0; e < 8; e++) acc[qi][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;            // of query head c, over this wave's keys so far
    const float soc = a.cap > 0.f ? a.scale / a.cap : 0.f;

    for (int tb = tb0; tb < t_end; tb += ROUND) {
        if (tb != tb0 || late) load_round(tb, kf, vf);
        // ---- scores of 16 keys for the group's query heads: lane (c, g) gets keys g*4 .. g*4+3 of head c ----------
        f32x4 s = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < DSTEPS; ks++) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[ks], qf[ks], s, 0, 0, 0);
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int t = tb + g * 4 + i;
            const bool ok = t >= lo && t < t_end;
            s[i] = ok ? score_of(s[i], a.scale, a.cap, soc) : -INFINITY;
            mx = fmaxf(mx, s[i]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        float alpha = 1.f, psum = 0.f;
        float pr[4] = {0.f, 0.f, 0.f, 0.f};
        if (m_new != -INFINITY) {
            alpha = __expf(m_run - m_new);
#pragma unroll
            for (int i = 0; i < 4; i++) { pr[i] = __expf(s[i] - m_new); psum += pr[i]; }
        }
        psum += __shfl_xor(psum, 16, 64);
        psum += __shfl_xor(psum, 32, 64);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (c < QT) {
#pragma unroll
            for (int i = 0; i < 4; i++) p_lds[wave][c][g * 4 + i] = pr[i];
            if (g == 0) alpha_lds[wave][c] = alpha;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // ---- weighted sum of the round's values -----------------------------------------------------------------------
#pragma unroll
        for (int qi = 0; qi < QT; qi++) {
            const float al = alpha_lds[wave][qi];
#pragma unroll
            for (int e = 0; e < 8; e++) acc[qi][e] *= al;
        }
#pragma unroll
        for (int j = 0; j < VPT; j++) {
            const int kk = kgw + j * KGW;
            if (kk < 16) {
                float vv[8];
#pragma unroll
                for (int e = 0; e < 8; e++) vv[e] = bf16_to_f32(vf[j].h[e]);
#pragma unroll
                for (int qi = 0; qi < QT; qi++) {
                    const float w = p_lds[wave][qi][kk];
#pragma unroll
                    for (int e = 0; e < 8; e++) acc[qi][e] = fmaf(w, vv[e], acc[qi][e]);
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    // ---- the four waves' results: rescale to a common maximum, add in wave and key-group order, write -------------
    if (c < QT && g == 0) { m_w[wave][c] = m_run; l_w[wave][c] = l_run; }
#pragma unroll
    for (int qi = 0; qi < QT; qi++) {
        if (qi >= G) continue;                       // G is the same for the whole block; unrolled, so that acc stays in registers
        if (pv_lane) {
#pragma unroll
            for (int e = 0; e < 8; e++) red[(wave * KGW + kgw) * HD + ch * 8 + e] = acc[qi][e];
        }
        __syncthreads();
        if (tid < HD) {
            float mx = -INFINITY;
            for (int w = 0; w < 4; w++) mx = fmaxf(mx, m_w[w][qi]);
            float num = 0.f, den = 0.f;
            for (int w = 0; w < 4; w++) {
                const float mw = m_w[w][qi];
                if (mw == -INFINITY) continue;
                const float f = __expf(mw - mx);
                float part = 0.f;
                for (int k2 = 0; k2 < KGW; k2++) part += red[(w * KGW + k2) * HD + tid];
                num += f * part;
                den += f * l_w[w][qi];
            }
            const int head = kvh * G + qi;
            if (a.nsplit == 1) {
                a.out[((size_t)seq * a.H + head) * HD + tid] = f32_to_bf16(num / den);
            } else {
                const size_t at = ((size_t)seq * a.H + head) * a.nsplit + split;
                a.ws_o[at * HD + tid] = num;
                if (tid == 0) { a.ws_ml[at * 2] = mx; a.ws_ml[at * 2 + 1] = den; }
            }
        }
        __syncthreads();
    }
}

// The slices of one (sequence, head): weights exp(m_s - max m) / sum, computed once by the first wave, then every
// thread adds its head elements in slice order.  Loads are unconditional (a slice without keys left its sum
// unwritten: its weight is zero and the value is replaced by zero).
__global__ void __launch_bounds__(256)
attn_decode_combine_k(const float* __restrict__ ws_o, const float* __restrict__ ws_ml, int nsplit,
                      bf16_t* __restrict__ out) {
    __shared__ float w_lds[128];
    const size_t at = (size_t)blockIdx.x * nsplit;               // blockIdx.x = sequence * heads + head
    const int tid = threadIdx.x;
    // the first 16 slices' sums are asked for before the weights are known: both come from memory at the same time
    constexpr int FIRST = 16;
    const int d = tid < HD ? tid : HD - 1;                       // the block has max(HD, 64) threads
    float o0[FIRST];
#pragma unroll
    for (int j = 0; j < FIRST; j++) o0[j] = ws_o[(at + (j < nsplit ? j : nsplit - 1)) * HD + d];
    if (tid < 64) {
        const int s0 = tid < nsplit ? tid : nsplit - 1, s1 = tid + 64 < nsplit ? tid + 64 : nsplit - 1;
        const float2 ml0 = *reinterpret_cast<const float2*>(ws_ml + (at + s0) * 2);
        const float2 ml1 = *reinterpret_cast<const float2*>(ws_ml + (at + s1) * 2);
        const float m0 = tid < nsplit ? ml0.x : -INFINITY, m1 = tid + 64 < nsplit ? ml1.x : -INFINITY;
        float mx = fmaxf(m0, m1);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        const float w0 = m0 == -INFINITY ? 0.f : __expf(m0 - mx), w1 = m1 == -INFINITY ? 0.f : __expf(m1 - mx);
        // the sum in slice order, so that it does not depend on how lanes are paired
        w_lds[tid] = w0 * ml0.y;
        w_lds[tid + 64] = w1 * ml1.y;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        float den = 0.f;
        for (int s = 0; s < nsplit; s++) den += w_lds[s];
        __builtin_amdgcn_wave_barrier();
        w_lds[tid] = w0 / den;
        w_lds[tid + 64] = w1 / den;
    }
    __syncthreads();
    float num = 0.f;
#pragma unroll
    for (int j = 0; j < FIRST; j++) {
        const float w = j < nsplit ? w_lds[j] : 0.f;
        num += w == 0.f ? 0.f : w * o0[j];
    }
    for (int s0 = FIRST; s0 < nsplit; s0 += 8) {
        float o[8], w[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int s = s0 + j < nsplit ? s0 + j : nsplit - 1;
            o[j] = ws_o[(at + s) * HD + d];
            w[j] = s0 + j < nsplit ? w_lds[s] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 8; j++) num += w[j] == 0.f ? 0.f : w[j] * o[j];
    }
    if (tid < HD) out[(size_t)blockIdx.x * HD + tid] = f32_to_bf16(num);
}

extern "C" long tp_attn_decode_workspace_floats(int n_seq, int H, int nsplit) {
    return nsplit > 1 ? (long)n_seq * H * nsplit * (HD + 2) : 0;
}

static int decode_launch(DecodeArgs a, int n_seq, void* workspace, hipStream_t s) {
    TP_REQUIRE(n_seq > 0 && a.H > 0 && a.KV > 0, "attention decode: empty shape");
    TP_REQUIRE(a.H % a.KV == 0, "attention: %d query heads are no multiple of %d kv heads", a.H, a.KV);
    const int G = a.H / a.KV;
    TP_REQUIRE(G <= 16, "attention decode (matrix-core kernel): %d query heads per kv head exceed 16", G);
    TP_REQUIRE(a.page >= 16 && (a.page & (a.page - 1)) == 0 && a.table_w > 0, "attention decode (matrix-core kernel): page size %d must be a power of two, at least 16", a.page);
    TP_REQUIRE(a.rows_cap == 0 || a.window <= a.rows_cap, "attention decode: a window of %d keys does not fit a ring of %d rows", a.window, a.rows_cap);
    TP_REQUIRE(a.rows_cap >= 0 && a.rows_cap % a.page == 0, "attention decode: ring of %d rows is no multiple of the page size %d", a.rows_cap, a.page);
    TP_REQUIRE(a.nsplit >= 1 && a.nsplit <= 128 && (a.nsplit == 1 || workspace), "attention decode: %d slices (at most 128) need a workspace", a.nsplit);
    TP_REQUIRE(a.KV <= 65535 && n_seq <= 65535, "attention decode: grid too large");
    if (a.nsplit > 1) {
        a.ws_o = (float*)workspace;
        a.ws_ml = a.ws_o + (size_t)n_seq * a.H * a.nsplit * HD;
    }
    dim3 grid(a.KV, n_seq, a.nsplit);
    if (G <= 1) attn_decode_k<1><<<grid, DTH, 0, s>>>(a);
    else if (G <= 2) attn_decode_k<2><<<grid, DTH, 0, s>>>(a);
    else if (G <= 4) attn_decode_k<4><<<grid, DTH, 0, s>>>(a);
    else if (G <= 8) attn_decode_k<8><<<grid, DTH, 0, s>>>(a);
    else attn_decode_k<16><<<grid, DTH, 0, s>>>(a);
    if (int rc = tp_check_launch("attention decode")) return rc;
    if (a.nsplit > 1) {
        attn_decode_combine_k<<<n_seq * a.H, HD < 64 ? 64 : HD, 0, s>>>(a.ws_o, a.ws_ml, a.nsplit, a.out);
        return tp_check_launch("attention decode (combine)");
    }
    return 0;
}

extern "C" int tp_attn_decode(const void* q, long q_stride, int n_seq, int H, int KV, const int* new_len,
                              const int* table, int table_w, const void* k_pool, const void* v_pool, int page,
                              int rows_cap, float scale, float cap, int window, void* out, void* workspace,
                              int nsplit, void* stream) {
    TP_REQUIRE(q_stride % 8 == 0 && (uintptr_t)q % 16 == 0, "attention decode: query rows must be 16-byte aligned");
    DecodeArgs a{(const bf16_t*)q, q_stride, H, KV, new_len, table, table_w, (bf16_t*)k_pool, (bf16_t*)v_pool,
                 page, rows_cap, scale, cap, window, (bf16_t*)out, nullptr, nullptr, nsplit,
                 nullptr, 0, 1, 0, 0, nullptr, 0, 0};
    return decode_launch(a, n_seq, workspace, (hipStream_t)stream);
}

// One launch for a decode step's rotation, cache write and attention: `qkv` holds each sequence's projections
// [heads | kv heads (keys) | kv heads (values)] x head size (queries only when write_kv is 0) as bf16 rows, or as
// float32 rows in n_slices K slices `slice_stride` elements apart.  Sequence i's new token has position new_len[i] - 1.
extern "C" int tp_attn_decode_fused(const void* qkv, int qkv_dtype, int n_slices, long slice_stride, long row_stride,
                                    const float* inv_freq, int rot, int write_kv,
                                    int n_seq, int H, int KV, const int* new_len, const int* table, int table_w,
                                    void* k_pool, void* v_pool, int page, int rows_cap, float scale, float cap,
                                    int window, void* out, void* workspace, int nsplit, void* stream) {
    TP_REQUIRE(qkv, "attention decode (fused): no projections");
    TP_REQUIRE(qkv_dtype == TP_BF16 || qkv_dtype == TP_F32, "attention decode (fused): projections of dtype %d", qkv_dtype);
    TP_REQUIRE(n_slices >= 1 && (n_slices == 1 || qkv_dtype == TP_F32), "attention decode (fused): %d slices must be float32", n_slices);
    TP_REQUIRE(rot >= 0 && rot <= HD && rot % 2 == 0, "attention decode (fused): rotary_dim %d must be even and at most head_dim %d", rot, HD);
    TP_REQUIRE(rot == 0 || inv_freq, "attention decode (fused): a rotation needs its frequency table");
    TP_REQUIRE(row_stride >= (long)(H + (write_kv ? 2 * KV : 0)) * HD, "attention decode (fused): rows of %ld elements are too short", row_stride);
    DecodeArgs a{nullptr, 0, H, KV, new_len, table, table_w, (bf16_t*)k_pool, (bf16_t*)v_pool,
                 page, rows_cap, scale, cap, window, (bf16_t*)out, nullptr, nullptr, nsplit,
                 qkv, qkv_dtype == TP_F32 ? 1 : 0, n_slices, slice_stride, row_stride, inv_freq, rot, write_kv};
    return decode_launch(a, n_seq, workspace, (hipStream_t)stream);
}
