// bf16 attention of a step's queries on the matrix cores, for one head size (compiled with -DTP_HD=<head_dim>, a
// multiple of 16 up to 256): every sequence brings `count` queries at its positions start .. start + count - 1
// and they attend over the positions before `start` where they lie, in the paged cache (through the page table:
// ring row p % rows_cap of a window's ring), and over the step's own rows of keys and values.
//
// Formula as the reference's attn_k (runtime/cuda/codebook_gemv.cu:240-270): score = (q . k) * scale, then
// cap * tanh(score / cap) if a cap is set, softmax over the visible keys in fp32, weighted sum of v, query head
// h reading kv head h / (heads / kv_heads); its multi-token form walks the cache in place from any position
// (runtime/cuda/codebook_gemv.cu:410-440).  The scale is an argument (rsqrt(head_dim) there), and a window W
// hides keys with p - t >= W (the reference has none: runtime/src/lib.rs:4455).
//
// Shape of the work.  A block owns one kv head of one sequence, up to four of that kv head's query heads and a
// run of query positions: its waves form CG column groups x KG key groups.  A column group is 32 query columns
// (one head x 32 positions), so that a tile of keys staged in LDS serves every head of the group that shares
// it; a key group takes every KG-th tile of 32 keys with a running softmax of its own, and the groups' states
// are joined through LDS at the end (a step of few query tiles gets its parallelism from the keys).
// Scores are computed transposed, S^T = K . Q^T, with v_mfma_f32_32x32x16_bf16: a key tile's rows are the A
// operand (one 16-byte LDS read per lane and instruction), the queries stay in registers as the B operand, and a
// lane ends up with 16 keys of ONE query: the softmax statistics are per-lane scalars (one exchange with lane
// ^ 32), and the probabilities, rounded to bf16, are the B operand of the second product as they lie.
// The second product is O^T = V^T . P^T.  V is staged as it is stored (row = key); its A operand (row = head
// element, 8 keys per lane) comes out of LDS through ds_read_b64_tr_b16, the transposing read of gfx950, so no
// transposed copy of V is ever made.
// K and V tiles travel global memory -> LDS directly (global_load_lds_dwordx4), each into a single buffer: the
// next K tile is asked for when every wave has multiplied the current one (in the middle of the softmax), the
// next V tile when every wave has used the current one, so that each load has about half a round to land and a
// round costs two barriers.  The first tiles are asked for before the queries.
//
// Measured on MI355X, Gemma-2 2B sizes (8 heads, 4 kv heads of 256, cap 50): 8 x 7,900 tokens 2.2 ms a layer
// (0.92 PFLOP/s; matrix pipes busy half the time, no LDS bank conflicts), 2,048 tokens 50 us.  What was tried and
// changed nothing there: fragments three and four ahead instead of two, a second chain of score accumulation,
// half or all of the queries in LDS, the block's upper waves running half a round behind the lower ones (slower:
// the halves differ in length and every wave waits for the slowest at both barriers).
#include "common.h"

#ifndef TP_HD
#error "compile with -DTP_HD=<head_dim>"
#endif

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 pf_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short pf_s16x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float pf_f32x16;

struct PrefillArgs {
    const bf16_t* q; long q_stride;
    const bf16_t* k; long k_stride; const bf16_t* v; long v_stride;     // the step's own rows
    const int* cu_rows;                       // [n_seq + 1]: rows of sequence s are cu_rows[s] .. cu_rows[s + 1] - 1
    const int* new_len;                       // [n_seq]: length after the step (first query at new_len - count); null: 0
    const int* table; int table_w;            // page table [n_seq, table_w] of the cache group
    const bf16_t* k_pool; const bf16_t* v_pool;
    int page_shift, page_mask, rows_cap;
    int H, KV, ghb_shift, pt_shift;           // heads of a kv head a block takes: 1 << ghb_shift; its position tiles: 1 << pt_shift
    int n_streams, pos_blocks;                // (sequence, kv head, head group) triples; blocks of positions per stream
    float scale, cap; int window;
    bf16_t* out;
};

namespace {
constexpr int HD = TP_HD;
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head_dim must be a multiple of 16 up to 256");
constexpr int KS16 = HD / 16;                 // k steps of the first product
constexpr int DT = (HD + 31) / 32;            // 32-row tiles of O^T
constexpr int KSUB = (HD + 63) / 64;          // sub-tiles of 64 head elements in LDS
constexpr int TILE_ELEMS = KSUB * 32 * 64;    // a K (or V) tile of 32 keys in LDS
constexpr int TILE_BYTES = TILE_ELEMS * 2;
constexpr int MERGE_LANE = DT * 16 + 4;       // floats a lane hands over: its part of O^T, maximum, sum (16-byte rows)
// At head size 256 the output (128 registers a lane) and the queries (64) leave too little room for fragments in
// flight: the last QL of a wave's query fragments live in LDS (1 KB each, one 16-byte read per lane and round).
constexpr int QL = HD > 128 ? 4 : 0, QR = KS16 - QL;
constexpr int KD = 2, VD = 2;                 // fragments of K (with the query fragment from LDS) and of V asked for ahead of their product
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LAZY = 8.f;                   // the running maximum moves only when a score exceeds it by this much (log 2 units)

// LDS layout of a tile: sub-tile j holds head elements 64 j .. 64 j + 63 as 32 rows (keys) of 128 bytes, whose
// 16-byte chunks sit at chunk ^ swizzle(key).  K is read by key rows (lanes 0..15 of a read: 16 keys, one chunk
// index): keys of one parity need 8 different places.  V is read by the transposing read, 4 keys x 64 bytes per 32
// lanes: keys 2 apart need different halves of the row.
__device__ __forceinline__ int swz_k(int key) { return (key >> 1) & 7; }
__device__ __forceinline__ int swz_v(int key) { return (((key >> 1) & 1) << 2) | ((key >> 2) & 3); }

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
// the other half-wave's value of x, combined with this one's (lanes l and l ^ 32 hold the same query)
__device__ __forceinline__ float pair_max(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ bf16_t bf16_bits(float f) {
    __bf16 b = (__bf16)f;
    return __builtin_bit_cast(bf16_t, b);
}
union PFrag { uint4 u; pf_bf16x8 v; pf_s16x4 h[2]; };

template <int CG, int KG> struct PrefillShape {
    static constexpr int THREADS = 64 * CG * KG;
    static constexpr size_t TILES = (size_t)2 * KG * TILE_BYTES + (size_t)CG * QL * 1024;      // K and V tiles, query fragments
    static constexpr size_t MERGE = KG > 1 ? (size_t)(KG / 2) * CG * 64 * MERGE_LANE * sizeof(float) : 0;
    static constexpr size_t LDS = TILES > MERGE ? TILES : MERGE;
    static_assert(LDS <= 160 * 1024, "a block's tiles must fit the LDS of a CU");
};
}  // namespace

// Registers: up to 256 a lane at head size 256 (two waves a SIMD); smaller heads need fewer, and a block of four
// waves then runs three to a SIMD (27B sizes, 2 x 7,900 tokens: 1.62 -> 1.42 ms; four to a SIMD spill and lose).
template <int CG, int KG, bool PAGED>
__global__ void __launch_bounds__(64 * CG * KG, (HD <= 128 && CG * KG == 4 ? 3 : 2))
attn_prefill_k(PrefillArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char prefill_lds[];
    bf16_t* const Kbuf = reinterpret_cast<bf16_t*>(prefill_lds);                  // [KG] tiles
    bf16_t* const Vbuf = Kbuf + KG * TILE_ELEMS;
    uint4* const Qbuf = reinterpret_cast<uint4*>(Vbuf + KG * TILE_ELEMS);         // [CG][QL][64 lanes]
    const int tid = threadIdx.x, lane = tid & 63, col = lane & 31, hi = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), kg = wave / CG, cg = wave % CG;

    // ---- which part of the step this block owns ---------------------------------------------------------------
    const int stream = blockIdx.x % a.n_streams, rank = blockIdx.x / a.n_streams;
    const int G = a.H / a.KV, HG = G >> a.ghb_shift;
    const int hg = stream % HG, kvh = (stream / HG) % a.KV, seq = stream / (HG * a.KV);
    const int PT = 1 << a.pt_shift, PB = 32 * PT;
    const int row0 = a.cu_rows[seq], Tq = a.cu_rows[seq + 1] - row0;
    const int q0 = (a.pos_blocks - 1 - rank) * PB;               // late positions see the most keys: they start first
    if (q0 >= Tq) return;
    const int start = PAGED ? a.new_len[seq] - Tq : 0, L = start + Tq;
    const int h = kvh * G + (hg << a.ghb_shift) + (cg >> a.pt_shift);
    const int qw0 = start + q0 + (cg & (PT - 1)) * 32;           // position of the wave's first query
    const int qpos = qw0 + col;
    const bool q_ok = qpos < L;

    // ---- the keys the block walks: tiles of 32 positions, aligned to multiples of 32 ---------------------------
    int k_lo = a.window > 0 ? max(0, start + q0 - a.window + 1) : 0;
    k_lo &= ~31;
    const int k_hi = min(L, start + q0 + PB);
    const int n_rounds = (k_hi - k_lo + 32 * KG - 1) / (32 * KG);

    // ---- loads of a tile: wave cg of the key group fetches the tile's key octets cg, cg + CG, ..; lane l the
    // 16-byte chunk that belongs at place (key l / 8 of the octet, place l % 8 of its 128-byte row) -----------------
    constexpr int NOCT = 4 / CG;
    const int ring_lo = PAGED && a.rows_cap > 0 ? k_lo % a.rows_cap : 0;
    const bf16_t* const k_rows = a.k + (size_t)kvh * HD;
    const bf16_t* const v_rows = a.v + (size_t)kvh * HD;
    auto row_of = [&](int key, const bf16_t*& kp, const bf16_t*& vp) {
        key = min(key, L - 1);                                    // past the end: a row that exists, hidden from every query
        if (PAGED && key < start) {
            int row = key;
            if (a.rows_cap > 0) {
                // key % rows_cap without a division: a cached key lies less than window + 30 positions behind k_lo (the
                // window's start rounded down to a tile), the window fits the ring and the ring has at least 16 rows,
                // so the sum below is less than four rings: three conditional subtractions
                row = ring_lo + (key - k_lo);
                row = row >= a.rows_cap ? row - a.rows_cap : row;
                row = row >= a.rows_cap ? row - a.rows_cap : row;
                row = row >= a.rows_cap ? row - a.rows_cap : row;
            }
            const int pg = a.table[(size_t)seq * a.table_w + (row >> a.page_shift)];
            const size_t at = ((((size_t)pg * a.KV + kvh) << a.page_shift) + (row & a.page_mask)) * HD;
            kp = a.k_pool + at;
            vp = a.v_pool + at;
        } else {
            const size_t r = (size_t)(row0 + key - start);
            kp = k_rows + r * a.k_stride;
            vp = v_rows + r * a.v_stride;
        }
    };
    // A load straight into LDS: lane l's 16 bytes land at dst + 16 l.  Written out as the instruction itself: told
    // of it, the compiler waits for every such load before the next LDS read of any address, which would undo the
    // overlap; the kernel waits for its loads where it has to (before the barrier that hands a tile over).
    auto dma = [&](const bf16_t* src, bf16_t* dst) {
        const unsigned at = (unsigned)(size_t)(__attribute__((address_space(3))) void*)dst;
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(src), "s"(at) : "memory");
    };
    const bf16_t* kp[NOCT];
    const bf16_t* vp[NOCT];
    auto rows_of_round = [&](int r) {
        const int kt = k_lo + 32 * (r * KG + kg);
#pragma unroll
        for (int o = 0; o < NOCT; o++) row_of(kt + (cg + o * CG) * 8 + (lane >> 3), kp[o], vp[o]);
    };
    auto issue_k = [&]() {
#pragma unroll
        for (int o = 0; o < NOCT; o++) {
            const int keyl = (cg + o * CG) * 8 + (lane >> 3), c = (lane & 7) ^ swz_k(keyl);
#pragma unroll
            for (int j = 0; j < KSUB; j++) {
                const int d = j * 64 + c * 8;
                dma(kp[o] + (d < HD ? d : 0), Kbuf + kg * TILE_ELEMS + (j * 32 + (cg + o * CG) * 8) * 64);
            }
        }
    };
    auto issue_v = [&]() {
#pragma unroll
        for (int o = 0; o < NOCT; o++) {
            const int keyl = (cg + o * CG) * 8 + (lane >> 3), c = (lane & 7) ^ swz_v(keyl);
#pragma unroll
            for (int j = 0; j < KSUB; j++) {
                const int d = j * 64 + c * 8;
                dma(vp[o] + (d < HD ? d : 0), Vbuf + kg * TILE_ELEMS + (j * 32 + (cg + o * CG) * 8) * 64);
            }
        }
    };

    // ---- where a lane reads its fragments --------------------------------------------------------------------------
    // K: key row `col`, head elements ks * 16 + hi * 8 ..: chunk ((ks & 3) << 1 | hi) of sub-tile ks >> 2
    const bf16_t* const Kt = Kbuf + kg * TILE_ELEMS + col * 64;
    int koff[4];
#pragma unroll
    for (int i = 0; i < 4; i++) koff[i] = (((i << 1) | hi) ^ swz_k(col)) << 3;
    // V through the transposing read: the 16 lanes of a quarter wave point at 4 keys x 4 pieces of 4 head elements and
    // get back, lane i, head element i of the quarter's 16 with its 4 keys.  Lane l: quarter b = l / 16 (head elements
    // (b & 1) * 16 .., keys hi * 4 ..), s = l % 16: key s / 4, piece s % 4.  Read u of k step t: keys 16 t + 8 u + hi * 4 + s / 4.
    const int vs = lane & 15, vkey = hi * 4 + (vs >> 2), vd = ((lane >> 4) & 1) * 16 + (vs & 3) * 4;   // + 16 t + 8 u; + 32 dt
    const bf16_t* const Vt = Vbuf + kg * TILE_ELEMS + vkey * 64 + (vd & 4);
    int voff[2][2];                                               // [dt & 1][u]
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int u = 0; u < 2; u++) voff[i][u] = ((((i * 32 + vd) >> 3) & 7) ^ swz_v(vkey + 8 * u)) << 3;

    pf_f32x16 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int e = 0; e < 16; e++) o[dt][e] = 0.f;
    float m_ref = -INFINITY, l_i = 0.f;                            // in units of log 2; l_i: this lane's 16 keys of every tile
    const float tanh_in = a.cap > 0.f ? 2.f * LOG2E * a.scale / a.cap : 0.f, cap2 = a.cap * LOG2E, scale2 = a.scale * LOG2E;
    const unsigned win = a.window > 0 ? (unsigned)a.window : 0x7fffffffu;

    rows_of_round(0);
    issue_k();
    issue_v();
    // ---- the wave's queries: B operand of the first product, in registers for the whole kernel -----------------
    // (the last QL of them in LDS, written by the column group's wave of key group 0)
    pf_bf16x8 qf[QR];
    uint4* const Qs = Qbuf + (cg * QL) * 64 + lane;
    {
        const bf16_t* qrow = a.q + (size_t)(row0 + (q_ok ? qpos : L - 1) - start) * a.q_stride + (size_t)h * HD + hi * 8;
#pragma unroll
        for (int ks = 0; ks < QR; ks++) qf[ks] = *reinterpret_cast<const pf_bf16x8*>(qrow + ks * 16);
        if (QL > 0 && kg == 0) {
#pragma unroll
            for (int ks = QR; ks < KS16; ks++) Qs[(ks - QR) * 64] = *reinterpret_cast<const uint4*>(qrow + ks * 16);
        }
    }

    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    float sc[16];                                    // lane: query `col`, keys kt + 8 (j / 4) + 4 hi + j % 4; in units of log 2
    for (int r = 0; r < n_rounds; r++) {
        const int kt = k_lo + 32 * (r * KG + kg);
        // wave-uniform: some key of the tile is visible to some query of the wave
        const bool visible = kt < k_hi && kt <= qw0 + 31 && qw0 < L && (a.window <= 0 || kt + 31 > qw0 - a.window);
        if (visible) {
            // two chains of accumulation where the registers allow it (at head size 256 they do not, and a second
            // chain measured no faster there: the SIMD's other wave fills in)
            constexpr bool TWO = KS16 > 1 && HD <= 128;
            pf_f32x16 s, s1;
#pragma unroll
            for (int e = 0; e < 16; e++) { s[e] = 0.f; s1[e] = 0.f; }
            PFrag kq[KD], qq[KD];                   // the fragments of k step ks in slot ks % KD
            auto k_frag = [&](int ks) {
                kq[ks % KD].u = *reinterpret_cast<const uint4*>(Kt + (ks >> 2) * (32 * 64) + koff[ks & 3]);
                if (ks >= QR) qq[ks % KD].u = Qs[(ks - QR) * 64];
            };
#pragma unroll
            for (int ks = 0; ks < KD - 1 && ks < KS16; ks++) k_frag(ks);
#pragma unroll
            for (int ks = 0; ks < KS16; ks++) {
                if (ks + KD - 1 < KS16) k_frag(ks + KD - 1);
                const pf_bf16x8 kf = kq[ks % KD].v, qv = ks < QR ? qf[ks < QR ? ks : 0] : qq[ks % KD].v;
                if (TWO && (ks & 1)) s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qv, s1, 0, 0, 0);
                else s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qv, s, 0, 0, 0);
            }
            if (TWO) s = s + s1;
            if (a.cap > 0.f) {                       // cap * tanh(x) = cap - 2 cap / (1 + e^(2x))
#pragma unroll
                for (int j = 0; j < 16; j++)
                    sc[j] = __builtin_fmaf(__builtin_amdgcn_rcpf(1.f + exp2_fast(s[j] * tanh_in)), -2.f * cap2, cap2);
            } else {
#pragma unroll
                for (int j = 0; j < 16; j++) sc[j] = s[j] * scale2;
            }
        }
        // The barrier stands in the middle of the softmax, so that both loads have about half a round to land: here
        // this round's V tile has landed and every wave has read the K tile, whose successor may come.
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (r + 1 < n_rounds) {
            rows_of_round(r + 1);
            issue_k();
        }
        if (visible) {
            const bool whole = kt + 31 <= qw0 && (a.window <= 0 || qw0 + 31 - kt < a.window);
            if (!whole) {
                const int d0 = qpos - kt - 4 * hi;   // distance to key j: d0 - 8 (j / 4) - j % 4; visible: 0 <= distance < window
#pragma unroll
                for (int j = 0; j < 16; j++)
                    sc[j] = (unsigned)(d0 - 8 * (j >> 2) - (j & 3)) < win ? sc[j] : -INFINITY;
            }
            float mx = sc[0];
#pragma unroll
            for (int j = 1; j < 16; j++) mx = fmaxf(mx, sc[j]);
            mx = pair_max(mx);
            const bool grow = mx > m_ref + LAZY;      // (never for a tile without a visible key: its maximum is -inf)
            const float m_new = grow ? mx : m_ref;
            if (__any(grow)) {
                const float alpha = grow ? exp2_fast(m_ref - m_new) : 1.f;
                l_i *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; dt++) o[dt] = o[dt] * alpha;
            }
            m_ref = m_new;
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            PFrag pf[2];
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const float p = exp2_fast(sc[j] - m_use);
                sum += p;
                pf[j >> 3].v[j & 7] = (__bf16)p;
            }
            l_i += sum;
            // fragment i = t * DT + dt of V^T (k step t, head elements dt * 32 ..): the next one is asked for before
            // this one is multiplied
            auto v_frag = [&](int i) {
                const int t = i / DT, dt = i % DT;
                PFrag vf;
                if (dt * 32 + 31 < HD) {
                    const bf16_t* base = Vt + (dt >> 1) * (32 * 64) + t * (16 * 64);
                    vf.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) pf_s16x4*)(base + voff[dt & 1][0]));
                    vf.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) pf_s16x4*)(base + 8 * 64 + voff[dt & 1][1]));
                } else {
                    // a last tile of 16 head elements: both quarters of a half-wave read them (rows past the head's end
                    // are never stored)
                    const int vdl = (vs & 3) * 4, c0 = ((dt * 32 + vdl) >> 3) & 7;
                    const bf16_t* base = Vbuf + kg * TILE_ELEMS + (dt >> 1) * (32 * 64) + (t * 16 + vkey) * 64 + (vdl & 4);
                    vf.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) pf_s16x4*)(base + ((c0 ^ swz_v(vkey)) << 3)));
                    vf.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) pf_s16x4*)(base + 8 * 64 + ((c0 ^ swz_v(vkey + 8)) << 3)));
                }
                return vf;
            };
            PFrag vq[VD];
#pragma unroll
            for (int i = 0; i < VD - 1 && i < 2 * DT; i++) vq[i % VD] = v_frag(i);
#pragma unroll
            for (int i = 0; i < 2 * DT; i++) {
                if (i + VD - 1 < 2 * DT) vq[(i + VD - 1) % VD] = v_frag(i + VD - 1);
                o[i % DT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vq[i % VD].v, pf[i / DT].v, o[i % DT], 0, 0, 0);
            }
        }
        // the next K tile has landed, and every wave has used the V tile, whose successor may come
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (r + 1 < n_rounds) issue_v();
    }

    // ---- the key groups' states join group 0's, pairwise, each rescaled to the common maximum --------------------
    if (KG > 1) {
        float* const merge = reinterpret_cast<float*>(prefill_lds);
#pragma unroll
        for (int half = KG / 2; half >= 1; half /= 2) {
            float* mine = merge + ((size_t)((kg - half) * CG + cg) * 64 + lane) * MERGE_LANE;
            float* theirs = merge + ((size_t)(kg * CG + cg) * 64 + lane) * MERGE_LANE;
            if (kg >= half && kg < 2 * half) {
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int e = 0; e < 16; e += 4)
                        *reinterpret_cast<float4*>(mine + dt * 16 + e) = make_float4(o[dt][e], o[dt][e + 1], o[dt][e + 2], o[dt][e + 3]);
                mine[DT * 16] = m_ref;
                mine[DT * 16 + 1] = l_i;
            }
            __syncthreads();
            if (kg < half) {
                const float mj = theirs[DT * 16], lj = theirs[DT * 16 + 1];
                const float m = fmaxf(m_ref, mj);
                const float a0 = m_ref == -INFINITY ? 0.f : exp2_fast(m_ref - m), aj = mj == -INFINITY ? 0.f : exp2_fast(mj - m);
                l_i = l_i * a0 + lj * aj;
                m_ref = m;
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int e = 0; e < 16; e += 4) {
                        const float4 t = *reinterpret_cast<const float4*>(theirs + dt * 16 + e);
                        o[dt][e] = o[dt][e] * a0 + t.x * aj;
                        o[dt][e + 1] = o[dt][e + 1] * a0 + t.y * aj;
                        o[dt][e + 2] = o[dt][e + 2] * a0 + t.z * aj;
                        o[dt][e + 3] = o[dt][e + 3] * a0 + t.w * aj;
                    }
            }
            __syncthreads();
        }
        if (kg > 0) return;
    }
    if (!q_ok) return;
    const float inv = 1.f / pair_sum(l_i);
    // lane: head elements dt * 32 + 8 (j / 4) + 4 hi + j % 4 of query `col`: four neighbours per store
    bf16_t* orow = a.out + ((size_t)(row0 + qpos - start) * a.H + h) * HD + 4 * hi;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int e = 0; e < 16; e += 4) {
            const int d = dt * 32 + 2 * e;            // 8 (e / 4)
            if (d + 4 * hi < HD) {
                ushort4 pk;
                pk.x = bf16_bits(o[dt][e] * inv); pk.y = bf16_bits(o[dt][e + 1] * inv);
                pk.z = bf16_bits(o[dt][e + 2] * inv); pk.w = bf16_bits(o[dt][e + 3] * inv);
                *reinterpret_cast<ushort4*>(orow + d) = pk;
            }
        }
}

namespace {
template <int CG, int KG, bool PAGED>
int prefill_launch(const PrefillArgs& a, int blocks, hipStream_t stream) {
    using Shape = PrefillShape<CG, KG>;
    static bool configured = false;                                   // more LDS than a kernel gets without asking
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_k<CG, KG, PAGED>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)Shape::LDS);
        if (e != hipSuccess) return tp_fail("attention prefill: cannot reserve %zu bytes of LDS: %s", (size_t)Shape::LDS, hipGetErrorString(e));
        configured = true;
    }
    attn_prefill_k<CG, KG, PAGED><<<blocks, Shape::THREADS, Shape::LDS, stream>>>(a);
    return 0;
}
}  // namespace

// q: M rows of queries, k and v: the same rows' keys and values (keys rotated), sequence s's at cu_rows[s] ..
// new_len (or null): the sequences' lengths after the step; what lies before a sequence's first row of the step is
// read from the cache (k_pool, v_pool [pages, kv_heads, page, head_dim] through `table`), as earlier steps left it.
// shape: 0 chooses by the size of the step; 1: blocks of 4 column groups, 2: 2 column groups x 4 key groups,
// 3: 2 column groups x 2 key groups (for tests and measurements).
extern "C" int tp_attn_prefill(const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride,
                               int M, int H, int KV, const int* cu_rows, int n_seq, int max_count,
                               const int* new_len, const int* table, int table_w, const void* k_pool, const void* v_pool,
                               int page, int rows_cap, float scale, float cap, int window, void* out, int shape, void* stream) {
    TP_REQUIRE(M > 0 && H > 0 && KV > 0 && n_seq > 0 && max_count > 0, "attention prefill: empty shape");
    TP_REQUIRE(H % KV == 0, "attention: %d query heads are no multiple of %d kv heads", H, KV);
    TP_REQUIRE(q_stride % 8 == 0 && k_stride % 8 == 0 && v_stride % 8 == 0 && (uintptr_t)q % 16 == 0 &&
               (uintptr_t)k % 16 == 0 && (uintptr_t)v % 16 == 0, "attention prefill: rows must be 16-byte aligned");
    TP_REQUIRE(scale > 0.f, "attention prefill: the scale %g must be positive", scale);
    const bool paged = new_len != nullptr;
    if (paged) {
        TP_REQUIRE(table && k_pool && v_pool && table_w > 0, "attention prefill: cached positions need the page table and the pools");
        TP_REQUIRE(page >= 16 && (page & (page - 1)) == 0, "attention prefill (matrix-core kernel): page size %d must be a power of two, at least 16", page);
        TP_REQUIRE(rows_cap >= 0 && rows_cap % page == 0, "attention prefill: ring of %d rows is no multiple of the page size %d", rows_cap, page);
        TP_REQUIRE(rows_cap == 0 || (window > 0 && window <= rows_cap), "attention prefill: a window of %d keys does not fit a ring of %d rows", window, rows_cap);
        TP_REQUIRE((uintptr_t)k_pool % 16 == 0 && (uintptr_t)v_pool % 16 == 0, "attention prefill: the pools must be 16-byte aligned");
    }
    const int G = H / KV;
    PrefillArgs a{};
    a.q = (const bf16_t*)q; a.q_stride = q_stride; a.k = (const bf16_t*)k; a.k_stride = k_stride; a.v = (const bf16_t*)v; a.v_stride = v_stride;
    a.cu_rows = cu_rows; a.new_len = new_len; a.table = table; a.table_w = table_w;
    a.k_pool = (const bf16_t*)k_pool; a.v_pool = (const bf16_t*)v_pool;
    int ps = 0;
    while (paged && (1 << ps) < page) ps++;
    a.page_shift = ps; a.page_mask = page - 1; a.rows_cap = paged ? rows_cap : 0;
    a.H = H; a.KV = KV; a.scale = scale; a.cap = cap; a.window = window; a.out = (bf16_t*)out;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    // heads of a kv head that share a block's tiles: the largest power of two that divides the group, up to the
    // block's column groups; the other column groups are further position tiles
    auto plan = [&](int cg, int& ghb_shift, int& pt_shift) {
        int gs = 0;
        while ((2 << gs) <= cg && G % (2 << gs) == 0) gs++;
        ghb_shift = gs;
        pt_shift = 0;
        while (((1 << gs) << (pt_shift + 1)) <= cg) pt_shift++;
    };
    // Blocks of 4 column groups share a staged tile among the most queries and run two (three) to a CU out of step
    // with one another: the choice where a step gives every CU four of them.  A smaller step gets its parallelism
    // from the keys: 2 column groups x 2 key groups, or, for sequences of a thousand tokens and more where even those
    // blocks are at most two a CU (at head sizes whose tiles let one 8-wave block fit a CU), 2 x 4: a quarter of the
    // rounds for the longest block.  Measured for 4x1 / 2x2 / 2x4: 2B sizes, 2,048 tokens 94 / 61 / 51 us, 4,096 tokens
    // 186 / 130 / 114, 8 x 512 tokens 34 / 27 / 36; 9B sizes, 2,048 tokens 100 / 72 / 69; 27B (heads of 128) 85 / 78 / 89.
    int cg = 4, kg = 1;
    {
        int gs, pts;
        plan(4, gs, pts);
        const long blocks4 = (long)tp_cdiv(max_count, 32 << pts) * n_seq * KV * (G >> gs);
        plan(2, gs, pts);
        const long blocks2 = (long)tp_cdiv(max_count, 32 << pts) * n_seq * KV * (G >> gs);
        if (shape == 0 && blocks4 < 4L * cus) shape = HD > 128 && blocks2 <= 2L * cus && max_count >= 1024 ? 2 : 3;
        if (shape == 2) { cg = 2; kg = 4; }
        if (shape == 3) { cg = 2; kg = 2; }
    }
    plan(cg, a.ghb_shift, a.pt_shift);
    a.n_streams = n_seq * KV * (G >> a.ghb_shift);
    a.pos_blocks = tp_cdiv(max_count, 32 << a.pt_shift);
    const long blocks = (long)a.n_streams * a.pos_blocks;
    TP_REQUIRE(blocks < (1L << 31), "attention prefill: %ld blocks exceed one launch", blocks);
    hipStream_t s = (hipStream_t)stream;
    int rc;
    if (cg == 4) rc = paged ? prefill_launch<4, 1, true>(a, (int)blocks, s) : prefill_launch<4, 1, false>(a, (int)blocks, s);
    else if (kg == 4) rc = paged ? prefill_launch<2, 4, true>(a, (int)blocks, s) : prefill_launch<2, 4, false>(a, (int)blocks, s);
    else rc = paged ? prefill_launch<2, 2, true>(a, (int)blocks, s) : prefill_launch<2, 2, false>(a, (int)blocks, s);
    if (rc) return rc;
    return tp_check_launch("attention prefill");
}
