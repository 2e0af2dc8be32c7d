// bf16 attention on the matrix cores for one head size (compiled with -DTP_HD=<head_dim>, a multiple of 16 up
// to 256): a prefill kernel over a buffer of keys and values (the step's own rows, behind the cached positions
// its queries still see when sequences continue) and a decode kernel over the paged cache.
//
// Formula as the reference's attn_k (runtime/cuda/codebook_gemv.cu:240-270): score = (q . k) * scale, then
// cap * tanh(score / cap) if a cap is set, softmax over the visible keys in fp32, weighted sum of v, query head
// h reading kv head h / (heads / kv_heads).  The scale is an argument (rsqrt(head_dim) in the reference), and a
// window W hides keys with p - t >= W (the reference has none: runtime/src/lib.rs:4455).
//
// Both kernels compute scores transposed, S^T = K . Q^T with v_mfma_f32_16x16x32_bf16: key rows are the A
// operand (a lane holds 8 consecutive elements of one key: one 16-byte load), queries the B operand, and a lane
// ends up with 4 keys of ONE query, so the softmax statistics are per-lane scalars and the probabilities are
// already laid out as the B operand of the second product.
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
// prefill: a sequence's keys and values are rows cu_keys[s] .. cu_keys[s + 1] - 1 of k and v, its queries the
// rows cu_rows[s] .. of q, and the queries are the sequence's LAST positions: with Tk keys and Tq queries the
// first query stands at key Tk - Tq (0 when every sequence starts in this step and the keys are its own rows;
// more when cached positions were gathered in front of them).  Only differences of positions count.
// Block = 64 or 32 queries of one (sequence, head); a wave owns 16 queries.  Key tiles of 32 go through LDS: K as
// stored (row = key), V transposed (row = head element) with the keys of a tile permuted so that a lane's 8
// probabilities meet the 8 values of the same keys in one 16-byte LDS read.
// =====================================================================================================
struct PrefillArgs {
    const bf16_t* q; long q_stride; const bf16_t* k; long k_stride; const bf16_t* v; long v_stride;
    int H, KV; const int* cu_rows; const int* cu_keys; float scale, cap; int window; bf16_t* out;
    const bf16_t* vt; long vt_rows;      // V transposed: [kv head][head element][padded key slot], vt_rows slots per row
};

namespace {
constexpr int BKV = 32;
// LDS layouts of a key tile, both in rows of 128 bytes whose 16-byte chunks sit at chunk ^ (row & 7): the 16 rows
// x 4 chunks that a fragment read touches then spread over the banks (padded rows lost 43 % of the LDS cycles to
// conflicts).  K: sub-tiles of 64 head elements, a row per key.  V transposed: two head elements per row, 32 key
// slots (64 bytes) each.
constexpr int KSUB = (HDP + 63) / 64;
__device__ __forceinline__ int k_at(int key, int d) {
    return (d >> 6) * (BKV * 64) + key * 64 + ((((d & 63) >> 3) ^ (key & 7)) << 3) + (d & 7);
}
__device__ __forceinline__ int v_at(int d, int slot_chunk) {
    return (d >> 1) * 64 + (((((d & 1) << 2) | slot_chunk) ^ ((d >> 1) & 7)) << 3);
}
}

// V of the step, transposed once per layer so that the attention blocks copy it into LDS as it lies:
// vt[kv head][d][slot], a sequence's keys in groups of 32 slots (its region padded to a multiple of 32), the keys
// of a group permuted as the second product's operand wants them (key a*16 + g*4 + b at slot g*8 + a*4 + b).
__device__ __forceinline__ int vt_base_of(const int* cu_rows, int seq) {
    int base = 0;
    for (int s = 0; s < seq; s++) base += (cu_rows[s + 1] - cu_rows[s] + BKV - 1) / BKV * BKV;
    return base;
}

__global__ void __launch_bounds__(256)
v_transpose_k(const bf16_t* __restrict__ v, long v_stride, int KV, const int* __restrict__ cu_rows,
              bf16_t* __restrict__ vt, long vt_rows) {
    __shared__ bf16_t tile[BKV][HD + 2];
    const int seq = blockIdx.z, kvh = blockIdx.y, kt = blockIdx.x * BKV;
    const int row0 = cu_rows[seq], T = cu_rows[seq + 1] - row0;
    if (kt >= T) return;
    const int base = vt_base_of(cu_rows, seq) + kt;
    for (int i = threadIdx.x; i < BKV * NCH; i += 256) {
        const int key = i / NCH, ch = i % NCH;
        Frag f;
        f.u = make_uint4(0, 0, 0, 0);
        if (kt + key < T) f.u = *reinterpret_cast<const uint4*>(v + (size_t)(row0 + kt + key) * v_stride + (size_t)kvh * HD + ch * 8);
#pragma unroll
        for (int e = 0; e < 8; e++) tile[key][ch * 8 + e] = f.h[e];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < HD * BKV; i += 256) {          // consecutive threads: consecutive slots of one d
        const int d = i / BKV, slot = i % BKV;
        const int key = ((slot >> 2) & 1) * 16 + (slot >> 3) * 4 + (slot & 3);   // slot g*8 + a*4 + b holds key a*16 + g*4 + b
        vt[((size_t)kvh * HD + d) * vt_rows + base + slot] = tile[key][d];
    }
}

// Block = 8 waves in PGROUPS groups of PWAVES, PQ queries of one (sequence, head): wave w of every group owns
// queries w*16 .. w*16+15.  Per round the block stages PGROUPS key tiles; group i takes the i-th, each group with its
// own running softmax, so the chain of dependent rounds is 1/PGROUPS as long as the keys; at the end the other groups
// hand (max, sum, unnormalised output) to group 0 through LDS.  A causal tile's work grows with its place in the
// sequence, and a block occupies a CU alone: the late (long) tiles of every head carry the lowest block ids, so the
// short ones fill in behind them, and a step of few tiles is cut into blocks of 32 queries instead of 64.
namespace {
constexpr int PTH = 512;                                         // threads of a prefill block
constexpr int KS_ELEMS = KSUB * BKV * 64, VT_ELEMS = HD * BKV;    // one tile's K and V^T in LDS
constexpr int MERGE_LANE = HD / 4 + 4;                           // a group's state per lane: its output tiles, max, sum (16-byte rows)
template <int PQ> struct PrefillShape {                          // PQ: queries of a block
    static constexpr int PWAVES = PQ / 16;                       // waves of a group
    static constexpr int PGROUPS = PTH / 64 / PWAVES;
    static constexpr int PKEYS = PGROUPS * BKV;                  // keys staged per round
    static constexpr int MERGE_GROUP = PWAVES * 64 * MERGE_LANE;
    static constexpr size_t TILE_BYTES = (size_t)PGROUPS * (KS_ELEMS + VT_ELEMS) * sizeof(bf16_t);
    static constexpr size_t MERGE_BYTES = (size_t)(PGROUPS - 1) * MERGE_GROUP * sizeof(float);
    static constexpr size_t LDS_BYTES = TILE_BYTES > MERGE_BYTES ? TILE_BYTES : MERGE_BYTES;
    static_assert(LDS_BYTES <= 160 * 1024, "a round's tiles must fit the LDS of a CU");
};
}

template <int PQ>
__global__ void __launch_bounds__(PTH)
attn_prefill_k(PrefillArgs a) {
    using Shape = PrefillShape<PQ>;
    constexpr int PWAVES = Shape::PWAVES, PGROUPS = Shape::PGROUPS, PKEYS = Shape::PKEYS, MERGE_GROUP = Shape::MERGE_GROUP;
    extern __shared__ __attribute__((aligned(16))) unsigned char prefill_lds[];
    bf16_t* Ks_all = reinterpret_cast<bf16_t*>(prefill_lds);                       // [group] tiles laid out by k_at
    bf16_t* Vt_all = Ks_all + PGROUPS * KS_ELEMS;                                  // [group] tiles laid out by v_at
    const int tid = threadIdx.x, grp = (tid >> 6) / PWAVES, wave = (tid >> 6) % PWAVES, lane = tid & 63, c = lane & 15, g = lane >> 4;
    const bf16_t* Ks = Ks_all + grp * KS_ELEMS;
    const bf16_t* Vt = Vt_all + grp * VT_ELEMS;
    // late query tiles see the most keys: they are given the low block ids, which start first
    const int seq = blockIdx.z, h = blockIdx.x % a.H, q0 = (gridDim.x / a.H - 1 - blockIdx.x / a.H) * PQ;
    // rows of the queries (row0, Tq of them) and of the keys (krow0, T of them); query i stands at key qofs + i
    const int row0 = a.cu_rows[seq], Tq = a.cu_rows[seq + 1] - row0;
    if (q0 >= Tq) return;
    const int krow0 = a.cu_keys[seq], T = a.cu_keys[seq + 1] - krow0, qofs = T - Tq;
    const int kvh = h / (a.H / a.KV);
    const int qw0 = qofs + q0 + wave * 16, qpos = qw0 + c;       // in key coordinates
    const bool q_ok = qpos < T;

    bf16x8 qf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
        const int d0 = ks * 32 + g * 8;
        qf[ks] = ld_frag(a.q + (size_t)(row0 + (q_ok ? qpos - qofs : 0)) * a.q_stride + (size_t)h * HD + d0, q_ok && d0 < HD);
    }
    if (HDP > HD)                                   // the padding columns of K stay zero for the whole kernel
        for (int i = tid; i < PKEYS * (HDP - HD); i += PTH) {
            const int key = i / (HDP - HD);
            Ks_all[(key / BKV) * KS_ELEMS + k_at(key % BKV, HD + i % (HDP - HD))] = 0;
        }

    f32x4 o[HD / 16];
#pragma unroll
    for (int dt = 0; dt < HD / 16; dt++) o[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m_i = -INFINITY, l_i = 0.f;                                // the running maximum in units of log 2
    constexpr float LOG2E = 1.4426950408889634f;
    const float tanh_in = a.cap > 0.f ? 2.f * LOG2E * a.scale / a.cap : 0.f, cap2 = a.cap * LOG2E, scale2 = a.scale * LOG2E;
    // the keys a lane's query sees: seen_lo .. seen_lo + seen_span
    const int seen_lo = a.window > 0 ? max(0, qpos - a.window + 1) : 0;
    const unsigned seen_span = (unsigned)max(0, min(qpos, T - 1) - seen_lo);

    int k_lo = a.window > 0 ? max(0, qofs + q0 - a.window + 1) : 0;
    k_lo &= ~(BKV - 1);
    const int k_hi = min(T, qofs + q0 + PQ);
    // a round's rows travel global memory -> registers (one round ahead, while the round before is being used) ->
    // LDS; K as stored, V from its transposed copy: HD rows of PKEYS slots per round
    constexpr int VCH = PKEYS / 8;                                  // 16-byte chunks of a head element's slots in a round
    constexpr int KTASKS = (PKEYS * NCH + PTH - 1) / PTH;           // (key, 16-byte chunk) per thread
    constexpr int VTASKS = (HD * VCH + PTH - 1) / PTH;              // (head element, chunk of its slots)
    bf16x8 fk[KTASKS], fv[VTASKS];
    // Addresses: a byte offset per thread from base pointers that are the same for the whole block and move with the
    // round (scalar work).  A chunk the round does not need reads the round's first chunk instead, so that every load
    // is issued without a branch and nothing is computed per round and lane but a comparison and a selection.
    constexpr bool K_EVEN = PTH % NCH == 0;                         // then task t's key is task 0's + t * PTH / NCH
    const char* const k_origin = reinterpret_cast<const char*>(a.k + (size_t)krow0 * a.k_stride + (size_t)kvh * HD);
    const char* const v_origin = reinterpret_cast<const char*>(a.vt + (size_t)kvh * HD * a.vt_rows + vt_base_of(a.cu_keys, seq));
    const size_t k_row_bytes = (size_t)a.k_stride * sizeof(bf16_t), v_row_bytes = (size_t)a.vt_rows * sizeof(bf16_t);
    unsigned koff[K_EVEN ? 1 : KTASKS];
    int kkey[K_EVEN ? 1 : KTASKS];
#pragma unroll
    for (int t = 0; t < (K_EVEN ? 1 : KTASKS); t++) {
        const int i = tid + t * PTH, key = i / NCH, ch = i % NCH;
        kkey[t] = i < PKEYS * NCH ? key : PKEYS;                    // PKEYS: no round needs it
        koff[t] = (unsigned)(key * (int)k_row_bytes + ch * 16);
    }
    const int v_d = tid / VCH, v_part = tid % VCH, v_tile_key = (v_part >> 2) * BKV;     // task t: head element v_d + t * PTH / VCH
    const unsigned voff = (unsigned)(v_d * (int)v_row_bytes + v_part * 16);
    auto fetch = [&](int kt) {
        const int left = min(k_hi - kt, PKEYS);                     // keys of the round that some query sees
        const char* const kb = k_origin + (size_t)kt * k_row_bytes;
        const char* const vb = v_origin + (size_t)kt * sizeof(bf16_t);
#pragma unroll
        for (int t = 0; t < KTASKS; t++) {
            unsigned off;
            if constexpr (K_EVEN) off = kkey[0] + t * (PTH / NCH) < left ? koff[0] + (unsigned)(t * (PTH / NCH)) * (unsigned)k_row_bytes : 0u;
            else off = kkey[t] < left ? koff[t] : 0u;
            fk[t] = *reinterpret_cast<const bf16x8*>(kb + off);
        }
#pragma unroll
        for (int t = 0; t < VTASKS; t++) {
            const bool need = v_d + t * (PTH / VCH) < HD && v_tile_key < left;      // a tile past the block's last key is never used
            fv[t] = *reinterpret_cast<const bf16x8*>(vb + (need ? voff + (unsigned)(t * (PTH / VCH)) * (unsigned)v_row_bytes : 0u));
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int t = 0; t < KTASKS; t++) {
            const int i = tid + t * PTH;
            const int key = i / NCH;
            if (i < PKEYS * NCH)
                *reinterpret_cast<bf16x8*>(Ks_all + (key / BKV) * KS_ELEMS + k_at(key % BKV, (i % NCH) * 8)) = fk[t];
        }
#pragma unroll
        for (int t = 0; t < VTASKS; t++) {
            const int i = tid + t * PTH;
            const int d = i / VCH, part = i % VCH;                   // slots part*8 .. +7 of the round: tile part / 4
            if (i < HD * VCH)
                *reinterpret_cast<bf16x8*>(Vt_all + (part >> 2) * VT_ELEMS + v_at(d, part & 3)) = fv[t];
        }
    };
    fetch(k_lo);
    for (int kr = k_lo; kr < k_hi; kr += PKEYS) {
        __syncthreads();                             // the round before has been used by every wave
        stage();
        __syncthreads();
        if (kr + PKEYS < k_hi) fetch(kr + PKEYS);
        const int kt = kr + grp * BKV;               // this group's tile
        const bool visible = kt < k_hi && qw0 < T && kt <= qw0 + 15 && !(a.window > 0 && kt + BKV - 1 < qw0 - a.window + 1);
        if (!visible) continue;                      // wave-uniform: every key of the tile is hidden from the wave's queries

        f32x4 s[2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            s[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ks++) {
                Frag kf;
                kf.u = *reinterpret_cast<const uint4*>(Ks + k_at(j * 16 + c, ks * 32 + g * 8));
                s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qf[ks], s[j], 0, 0, 0);
            }
        }
        // A lane holds the scores of keys kt + j*16 + g*4 + i for its query qpos.  From here on they are in units of
        // log 2 (the constants carry the factor), so that every exponential is one instruction; the branches are the
        // same for the whole wave.
        float sc[8];
        if (a.cap > 0.f) {                           // cap * tanh(x) = cap - 2 cap / (1 + e^(2x))
#pragma unroll
            for (int e = 0; e < 8; e++)
                sc[e] = __builtin_fmaf(__builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(s[e >> 2][e & 3] * tanh_in)), -2.f * cap2, cap2);
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) sc[e] = s[e >> 2][e & 3] * scale2;
        }
        // a tile every query of the wave sees whole needs no mask
        const bool whole = kt + BKV - 1 <= qw0 && qw0 + 15 < T && (a.window <= 0 || qw0 + 15 - kt < a.window);
        if (!whole) {
            const int first = kt + g * 4 - seen_lo;
#pragma unroll
            for (int e = 0; e < 8; e++)
                sc[e] = (unsigned)(first + (e >> 2) * 16 + (e & 3)) <= seen_span ? sc[e] : -INFINITY;
        }
        float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_i, mx);
        const float m_ref = m_new == -INFINITY ? 0.f : m_new;      // a query that has seen no key yet: every term is 0
        const float alpha = m_i == m_new ? 1.f : __builtin_amdgcn_exp2f(m_i - m_ref);
        float sum = 0.f;
        Frag pf;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float p = __builtin_amdgcn_exp2f(sc[e] - m_ref);
            sum += p;
            pf.h[e] = bf16_bits(p);
        }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        l_i = l_i * alpha + sum;
        m_i = m_new;
        if (__any(alpha != 1.f)) {                   // once the running maxima settle, nothing to rescale
#pragma unroll
            for (int dt = 0; dt < HD / 16; dt++) o[dt] = o[dt] * alpha;
        }
#pragma unroll
        for (int dt = 0; dt < HD / 16; dt++) {
            Frag vf;
            vf.u = *reinterpret_cast<const uint4*>(Vt + v_at(dt * 16 + c, g));
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf.v, o[dt], 0, 0, 0);
        }
    }
    // ---- the other groups' states join group 0's, in the groups' order, all rescaled to the common maximum ---------
    __syncthreads();                                 // the tiles in LDS are done with
    float* merge = reinterpret_cast<float*>(prefill_lds) + (size_t)(wave * 64 + lane) * MERGE_LANE;
    if (grp > 0) {
        float* mine = merge + (size_t)(grp - 1) * MERGE_GROUP;
#pragma unroll
        for (int dt = 0; dt < HD / 16; dt++) *reinterpret_cast<f32x4*>(mine + dt * 4) = o[dt];
        mine[HD / 4] = m_i;
        mine[HD / 4 + 1] = l_i;
    }
    __syncthreads();
    if (grp > 0 || !q_ok) return;
    float m = m_i;
#pragma unroll
    for (int j = 0; j < PGROUPS - 1; j++) m = fmaxf(m, merge[(size_t)j * MERGE_GROUP + HD / 4]);
    const float a0 = m_i == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_i - m);
    float l = l_i * a0;
#pragma unroll
    for (int dt = 0; dt < HD / 16; dt++) o[dt] = o[dt] * a0;
#pragma unroll
    for (int j = 0; j < PGROUPS - 1; j++) {
        const float* theirs = merge + (size_t)j * MERGE_GROUP;
        const float mj = theirs[HD / 4];
        const float aj = mj == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mj - m);
        l += theirs[HD / 4 + 1] * aj;
#pragma unroll
        for (int dt = 0; dt < HD / 16; dt++) o[dt] = o[dt] + *reinterpret_cast<const f32x4*>(theirs + dt * 4) * aj;
    }
    const float inv = 1.f / l;
    bf16_t* orow = a.out + ((size_t)(row0 + qpos - qofs) * a.H + h) * HD;
#pragma unroll
    for (int dt = 0; dt < HD / 16; dt++) {
        ushort4 pk;
        pk.x = bf16_bits(o[dt][0] * inv); pk.y = bf16_bits(o[dt][1] * inv);
        pk.z = bf16_bits(o[dt][2] * inv); pk.w = bf16_bits(o[dt][3] * inv);
        *reinterpret_cast<ushort4*>(orow + dt * 16 + g * 4) = pk;
    }
}

template <int PQ>
static int prefill_launch(const PrefillArgs& a, int max_count, int H, int n_seq, hipStream_t stream) {
    constexpr size_t lds = PrefillShape<PQ>::LDS_BYTES;
    static bool configured = false;                                   // more LDS than a kernel gets without asking
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_k<PQ>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return tp_fail("attention prefill: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        configured = true;
    }
    attn_prefill_k<PQ><<<dim3(tp_cdiv(max_count, PQ) * H, 1, n_seq), PTH, lds, stream>>>(a);
    return 0;
}

// elements of the transposed copy of V the prefill kernel needs as workspace (Mk: rows of keys)
extern "C" long tp_attn_prefill_workspace_elems(int Mk, int KV, int n_seq) {
    return (long)KV * HD * ((long)Mk + (long)BKV * n_seq + BKV);
}

// q: M rows of queries, sequence s's at cu_rows[s] ..; k, v: Mk rows of keys and values, sequence s's at
// cu_keys[s] .. (null: the queries' own rows, cu_rows); a sequence's queries are its last positions.
extern "C" int tp_attn_prefill(const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride,
                               int M, int H, int KV, const int* cu_rows, int n_seq, int max_count,
                               const int* cu_keys, int Mk, int max_keys,
                               float scale, float cap, int window, void* out, void* workspace, void* stream) {
    TP_REQUIRE(M > 0 && H > 0 && KV > 0 && n_seq > 0 && max_count > 0, "attention prefill: empty shape");
    TP_REQUIRE(H % KV == 0, "attention: %d query heads are no multiple of %d kv heads", H, KV);
    if (!cu_keys) { cu_keys = cu_rows; Mk = M; max_keys = max_count; }
    TP_REQUIRE(Mk >= M && max_keys >= max_count, "attention prefill: %d keys (at most %d a sequence) for %d queries (at most %d)", Mk, max_keys, M, max_count);
    TP_REQUIRE(q_stride % 8 == 0 && k_stride % 8 == 0 && v_stride % 8 == 0 && (uintptr_t)q % 16 == 0 &&
               (uintptr_t)k % 16 == 0 && (uintptr_t)v % 16 == 0, "attention prefill: rows must be 16-byte aligned");
    TP_REQUIRE(n_seq <= 65535 && (long)tp_cdiv(max_count, 32) * H < (1L << 31), "attention prefill: %d heads / %d sequences exceed one launch", H, n_seq);
    TP_REQUIRE(workspace && (uintptr_t)workspace % 16 == 0, "attention prefill: needs its 16-byte aligned workspace");
    TP_REQUIRE(k_stride < (1L << 22) && (long)HD * ((long)Mk + (long)BKV * n_seq + BKV) < (1L << 30),
               "attention prefill: %d rows of stride %ld exceed the kernel's 32-bit offsets", Mk, k_stride);
    TP_REQUIRE(KV <= 65535, "attention prefill: %d kv heads exceed one launch", KV);
    const long vt_rows = (long)Mk + (long)BKV * n_seq + BKV;        // every sequence's region is padded to whole groups
    v_transpose_k<<<dim3(tp_cdiv(max_keys, BKV), KV, n_seq), 256, 0, (hipStream_t)stream>>>(
        (const bf16_t*)v, v_stride, KV, cu_keys, (bf16_t*)workspace, vt_rows);
    if (int rc = tp_check_launch("attention prefill (transpose of V)")) return rc;
    PrefillArgs a{(const bf16_t*)q, q_stride, (const bf16_t*)k, k_stride, (const bf16_t*)v, v_stride, H, KV, cu_rows, cu_keys,
                  scale, cap, window, (bf16_t*)out, (const bf16_t*)workspace, vt_rows};
    // 64 queries a block stage each key once per 64 queries; 32 a block make twice the blocks, for grids that would
    // not give every CU a block of 64 (measured, 8 heads of 256: 26 against 30 us at 512 tokens, 75 against 84 at
    // 2,048, but 151 against 121 at 3,072; 32 heads of 128 at 2,048 tokens: 145 against 89 us)
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    const bool small = (long)tp_cdiv(max_count, 64) * H * n_seq <= cus;
    if (int rc = small ? prefill_launch<32>(a, max_count, H, n_seq, (hipStream_t)stream)
                       : prefill_launch<64>(a, max_count, H, n_seq, (hipStream_t)stream)) return rc;
    return tp_check_launch("attention prefill");
}

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
