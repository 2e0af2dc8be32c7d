// bf16 product for many rows (prefill) and for few rows of a wide or large matrix: LDS-tiled, on the matrix cores,
// fp32 accumulation.
//
// Block: 256 threads = 4 waves in a 2 x 2 arrangement over a tile of Y (128 x 128, 128 x 96, 128 x 256 or 64 x 64; 4 x 1 over 64 x 32); each
// wave owns TM x TN tiles of v_mfma_f32_16x16x32_bf16.  W rows are the A operand and X rows the B operand (both are
// contiguous along k, which is what the instruction wants per lane), so a lane ends up with 4 consecutive columns of
// one row of Y (one 8- or 16-byte store), and with the gate and the up column of the same unit in two accumulators of
// the same lane (the packed gate/up matrix alternates 16 gate rows and 16 up rows).
// K is walked in steps through one LDS buffer (three blocks fit a CU).  Two loops: gemm_mfma_direct_k loads a step's
// tile from global memory straight into LDS while the step before is multiplied out of registers; gemm_mfma_k issues
// the next step's global loads into registers before the current step's products and writes them to LDS after them
// (any K, any tile).  The 16-byte chunks of an LDS row are stored at chunk ^ (row & 7) (rows of 128 bytes; ^ (row & 15)
// in rows of 256), so that the 16 rows a fragment read touches spread over the banks (measured: bank conflicts fall
// from a third of the LDS cycles with padded rows to a few per cent).
// Consecutive block ids walk the M tiles of one N tile, so blocks in flight together share W tiles (large grids:
// per XCD, see the kernel).
#include "gemm.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

namespace {
constexpr int BK = 64;                                        // k step of the large tiles; LDS rows are one step long, unpadded
// k step of the 64 x 64 tiles.  They stream W, and what a block has in flight is one step of its tile: with steps of
// 64 the 288 blocks of the 2B gate/up product hold 2.4 MB between them, too little to keep HBM busy (cold weights,
// 64 rows: 34.6 us; steps of 128: 26.4 us; steps of 256: 26.3 us, and the smaller products lose).
constexpr int SMALL_KS = 128;
union Frag { uint4 u; bf16x8 v; };
// The value as it is, in a vector register the compiler takes to be new: an address 'block-wide pointer + this' then
// stays a scalar base with a 32-bit lane offset, instead of a 64-bit pointer per lane that is kept and moved along.
__device__ __forceinline__ unsigned in_register(unsigned v) {
    asm volatile("" : "+v"(v));
    return v;
}
}

// A wave's accumulators to Y.  The lane holds Y[m = .. + r][n = .. + g*4 + v], v = 0..3: four neighbours of a row go
// out in one store where the row length allows the alignment.
template <int EPI, int TM, int TN>
__device__ __forceinline__ void store_tile(const f32x4 (&acc)[TM][TN], void* __restrict__ Y, int M, int N, int m0, int n0,
                                           int wm, int wn, int r, int g, int out_dtype, float2 epi, int units) {
    const int width = EPI == TP_EPI_GATED ? units : N;
    const bool wide = (width & 3) == 0;
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int m = m0 + wm * 16 * TM + i * 16 + r;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; j += (EPI == TP_EPI_GATED ? 2 : 1)) {
            float o[4];
            int col;                                            // first of the four columns of Y (units if gated)
            if (EPI == TP_EPI_GATED) {
                col = ((n0 + wn * 16 * TN + j * 16) >> 1) + g * 4;
#pragma unroll
                for (int v = 0; v < 4; v++) o[v] = gate_act_fast(acc[i][j][v], epi) * acc[i][j + 1 < TN ? j + 1 : j][v];
            } else {
                col = n0 + wn * 16 * TN + j * 16 + g * 4;
#pragma unroll
                for (int v = 0; v < 4; v++) o[v] = EPI == TP_EPI_SOFTCAP ? softcap_f(acc[i][j][v], epi.x) : acc[i][j][v];
            }
            if (col >= width) continue;
            const size_t at = (size_t)m * width + col;
            if (wide) {                                         // width % 4 == 0 and col % 4 == 0: all four are inside
                if (out_dtype == TP_F32) *reinterpret_cast<f32x4*>((float*)Y + at) = (f32x4){o[0], o[1], o[2], o[3]};
                else {
                    ushort4 pk;
                    pk.x = f32_to_bf16(o[0]); pk.y = f32_to_bf16(o[1]); pk.z = f32_to_bf16(o[2]); pk.w = f32_to_bf16(o[3]);
                    *reinterpret_cast<ushort4*>((bf16_t*)Y + at) = pk;
                }
            } else {
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    if (col + v >= width) break;
                    if (out_dtype == TP_F32) ((float*)Y)[at + v] = o[v];
                    else ((bf16_t*)Y)[at + v] = f32_to_bf16(o[v]);
                }
            }
        }
    }
}

// TM x TN: the 16 x 16 tiles of a wave; the block's 2 x 2 waves cover BM = 32 TM rows of X and BN = 32 TN rows of W
// WM: waves along the rows of X (2: the 2 x 2 arrangement; 4: four waves over 64 rows of X, one wave across the tile's rows of W)
// DEEP: two k steps are asked for ahead, in two sets of staging registers (tiles that stream W for few rows)
// SHORT: whole tiles load their k steps by the short path described below
// KS: elements of a k step (64, or 128 for the 64 x 64 tiles, which stream W and are bound by the bytes a block has
// in flight: one step ahead is all a block asks for)
template <int EPI, int TM, int TN, bool SHORT, int KS = BK, int WM = 2, bool DEEP = false>
__global__ void __launch_bounds__(256, 2)
gemm_mfma_k(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, void* __restrict__ Y,
            int M, int N, int K, int m_tiles, int out_dtype, float2 epi, int units, int k_per_split, int xcd_panels) {
    constexpr int WN = 4 / WM, BM = 16 * WM * TM, BN = 16 * WN * TN, BK = KS, LDS = KS, CPR = KS / 8;
    constexpr int LA = BM * KS / 2048, LB = BN * KS / 2048;    // 16-byte chunks of a step's tile per thread
    static_assert(BM * KS % 2048 == 0 && BN * KS % 2048 == 0, "a step's tile is a whole number of chunks per thread");
    constexpr int SWZ = CPR >= 16 ? 15 : 7;        // rows 256 bytes long all start at one bank: their 16 chunks are permuted as a whole
    static_assert(!SHORT || (KS == 64 && WM == 2), "the short load path is written for steps of 64 and 2 x 2 waves");
    __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDS];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * LDS];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wm = WM == 4 ? wave : wave >> 1, wn = WM == 4 ? 0 : wave & 1;
    // Block ids go to the chip's 8 XCDs in turn, and each XCD has an L2 of its own.  On a large grid an XCD therefore
    // takes a contiguous range of the tiles, walked in panels of four N tiles (M tiles of a panel one after another, its
    // N tiles fastest), so that the blocks an XCD runs together share their W and X tiles in its L2.  Measured on the
    // 2B gate/up product at 2,048 rows (2,304 tiles): a tenth on a plain product that writes all of Y, two per cent
    // with the gated epilogue; up to some hundred tiles nothing.
    int vb = blockIdx.x, mt, nt;
    if (xcd_panels) {
        const int total = gridDim.x, base = total >> 3, rem = total & 7, xcd = vb & 7;
        vb = xcd * base + min(xcd, rem) + (vb >> 3);
        const int n_tiles = total / m_tiles, per_panel = 4 * m_tiles, p = vb / per_panel, q = vb - p * per_panel;
        const int width = min(4, n_tiles - p * 4);
        nt = p * 4 + q % width;
        mt = q / width;
    } else {
        mt = vb % m_tiles;
        nt = vb / m_tiles;
    }
    const int m0 = mt * BM, n0 = nt * BN;
    // a K slice per blockIdx.y: slices go to Y as float32 [slices, M, N] for the consumer to add in slice order
    const int k_begin = blockIdx.y * k_per_split;
    const int k_end = min(K, k_begin + k_per_split);
    if (gridDim.y > 1) Y = (float*)Y + (size_t)blockIdx.y * M * N;

    // global -> register staging: TM (TN) chunks of 16 bytes per thread and operand; chunk c = tid + 256 i: row c / 8,
    // k chunk c % 8.  A whole k step of a whole tile is loaded without a branch or an address computed per lane: the
    // lane's chunk 0 lies at one byte offset, fixed for the kernel, from base pointers that are the same for the whole
    // block (32 rows on per chunk, 64 elements on per step: scalar work).  A tile over the edge of Y computes a clamped
    // row per chunk; only a last, partial step tests every chunk.  A launch without a whole tile (fewer rows than a tile has) and the 64 x 64 tiles,
    // which stream W, run without the short path compiled in: its mere presence costs them a fifth (27B gate/up at 64
    // rows in 128 x 128 tiles: 188 against 149 us), while whole large tiles gain a twentieth from it.
    constexpr int SETS = DEEP ? 2 : 1;             // register sets of staged chunks: k steps asked for ahead
    bf16x8 ra[SETS][LA], rb[SETS][LB];
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const bool inner = SHORT && m0 + BM <= M && n0 + BN <= N;
    const unsigned xoff = (unsigned)(tid >> 3) * (unsigned)K * 2u + (unsigned)(tid & 7) * 16u;      // the same for X and W
    const size_t rows32 = (size_t)32 * K * 2;
    const char* const x_origin = reinterpret_cast<const char*>(X + (size_t)m0 * K);
    const char* const w_origin = reinterpret_cast<const char*>(W + (size_t)n0 * K);
    auto fetch = [&](bf16x8 (&ra)[LA], bf16x8 (&rb)[LB], int k0) {
        if (inner && k0 + BK <= k_end) {
            const char* const xb = x_origin + (size_t)k0 * 2, * const wb = w_origin + (size_t)k0 * 2;
            const unsigned off = in_register(xoff);
#pragma unroll
            for (int i = 0; i < LA; i++) ra[i] = *reinterpret_cast<const bf16x8*>(xb + i * rows32 + off);
#pragma unroll
            for (int i = 0; i < LB; i++) rb[i] = *reinterpret_cast<const bf16x8*>(wb + i * rows32 + off);
        } else if (SHORT && k0 + BK <= k_end) {
            // a tile over the edge of Y: a row past the edge reads the tile's last row (its products are never stored)
            const char* const xb = x_origin + (size_t)k0 * 2, * const wb = w_origin + (size_t)k0 * 2;
            const unsigned chunk = in_register((unsigned)(tid & 7) * 16u), row_bytes = (unsigned)K * 2u;
#pragma unroll
            for (int i = 0; i < LA; i++)
                ra[i] = *reinterpret_cast<const bf16x8*>(xb + ((unsigned)min((tid >> 3) + 32 * i, M - 1 - m0) * row_bytes + chunk));
#pragma unroll
            for (int i = 0; i < LB; i++)
                rb[i] = *reinterpret_cast<const bf16x8*>(wb + ((unsigned)min((tid >> 3) + 32 * i, N - 1 - n0) * row_bytes + chunk));
        } else {
#pragma unroll
            for (int i = 0; i < LA; i++) {
                const int c = tid + i * 256, row = c / CPR, k = k0 + (c % CPR) * 8, m = m0 + row;
                ra[i] = (m < M && k < k_end) ? *reinterpret_cast<const bf16x8*>(X + (size_t)m * K + k) : zero;
            }
#pragma unroll
            for (int i = 0; i < LB; i++) {
                const int c = tid + i * 256, row = c / CPR, k = k0 + (c % CPR) * 8, n = n0 + row;
                rb[i] = (n < N && k < k_end) ? *reinterpret_cast<const bf16x8*>(W + (size_t)n * K + k) : zero;
            }
        }
    };
    auto stage = [&](const bf16x8 (&ra)[LA], const bf16x8 (&rb)[LB]) {
#pragma unroll
        for (int i = 0; i < LA; i++) {
            const int c = tid + i * 256, row = c / CPR, kc = ((c % CPR) ^ (row & SWZ)) * 8;  // chunk j of a row sits at j ^ (row & SWZ)
            *reinterpret_cast<bf16x8*>(As + row * LDS + kc) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < LB; i++) {
            const int c = tid + i * 256, row = c / CPR, kc = ((c % CPR) ^ (row & SWZ)) * 8;
            *reinterpret_cast<bf16x8*>(Bs + row * LDS + kc) = rb[i];
        }
    };

    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    auto products = [&]() {
#pragma unroll
        for (int ks = 0; ks < BK; ks += 32) {
            Frag a[TM], b[TN];
            const int kc = (((ks >> 3) + g) ^ (r & SWZ)) * 8;
#pragma unroll
            for (int i = 0; i < TM; i++) a[i].u = *reinterpret_cast<const uint4*>(As + (wm * 16 * TM + i * 16 + r) * LDS + kc);
#pragma unroll
            for (int j = 0; j < TN; j++) b[j].u = *reinterpret_cast<const uint4*>(Bs + (wn * 16 * TN + j * 16 + r) * LDS + kc);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[j].v, a[i].v, acc[i][j], 0, 0, 0);
        }
    };
    // one step: the set's chunks to LDS, the set refilled `SETS` steps ahead, the step's products
    auto step = [&](bf16x8 (&ra)[LA], bf16x8 (&rb)[LB], int k0) {
        __syncthreads();                       // everyone is done reading the previous tile
        stage(ra, rb);
        __syncthreads();
        if (k0 + SETS * BK < k_end) fetch(ra, rb, k0 + SETS * BK);
        products();
    };

    fetch(ra[0], rb[0], k_begin);
    if (DEEP && k_begin + BK < k_end) fetch(ra[SETS - 1], rb[SETS - 1], k_begin + BK);
    for (int k0 = k_begin; k0 < k_end; k0 += SETS * BK) {
        step(ra[0], rb[0], k0);
        if (DEEP && k0 + BK < k_end) step(ra[SETS - 1], rb[SETS - 1], k0 + BK);
    }

    store_tile<EPI, TM, TN>(acc, Y, M, N, m0, n0, wm, wn, r, g, out_dtype, epi, units);
}

// The loop of the large tiles (128 x 128 and 128 x 96) when K is a multiple of 64: the k step's tile comes from
// global memory straight into LDS (global_load_lds_dwordx4: no staging registers, no LDS write instructions).  One LDS
// buffer, as above, so that three blocks fit a CU: a step reads all its fragments into registers, a barrier, then the
// loads of the next step are issued into the same buffer and fly while the step's 32 matrix instructions run; a
// second barrier when they have landed.  A lane's place in LDS is fixed by its lane number (16 bytes on from its
// neighbour's), so the swizzle is applied on the global side: the lane whose place is (row, j) fetches chunk
// j ^ (row & 7) of that row.  Rows past the edge of Y fetch the last row (their products are never stored).
// Measured at the 2B shapes against the register-staged loop: gate/up at 2,048 rows 185 -> 155 us (1.1 PFLOP/s), at
// 8,192 rows 660 (128 x 256 tiles) -> 632 us; qkv at 2,048 rows 52 -> 42 us; down, unsliced, 133 -> 125 us.
// (Two LDS buffers with one barrier a step were no faster and leave two blocks a CU.)
template <int EPI, int TN>
__global__ void __launch_bounds__(256, 2)
gemm_mfma_direct_k(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, void* __restrict__ Y,
                   int M, int N, int K, int m_tiles, int out_dtype, float2 epi, int units, int k_per_split, int xcd_panels) {
    constexpr int TM = 4, BM = 128, BN = 32 * TN, LDS = BK;
    __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDS];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * LDS];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;
    int vb = blockIdx.x, mt, nt;                     // the order of the tiles: as in gemm_mfma_k
    if (xcd_panels) {
        const int total = gridDim.x, base = total >> 3, rem = total & 7, xcd = vb & 7;
        vb = xcd * base + min(xcd, rem) + (vb >> 3);
        const int n_tiles = total / m_tiles, per_panel = 4 * m_tiles, p = vb / per_panel, q = vb - p * per_panel;
        const int width = min(4, n_tiles - p * 4);
        nt = p * 4 + q % width;
        mt = q / width;
    } else {
        mt = vb % m_tiles;
        nt = vb / m_tiles;
    }
    const int m0 = mt * BM, n0 = nt * BN;
    const int k_begin = blockIdx.y * k_per_split;
    const int k_end = min(K, k_begin + k_per_split);
    if (gridDim.y > 1) Y = (float*)Y + (size_t)blockIdx.y * M * N;

    // load i of a thread: row (tid >> 3) + 32 i of the tile, the chunk that belongs at the lane's place
    const int srow = tid >> 3, chunk = (lane & 7) ^ (srow & 7);
    unsigned xo[TM], wo[TN];
#pragma unroll
    for (int i = 0; i < TM; i++) xo[i] = (unsigned)min(m0 + srow + 32 * i, M - 1) * (unsigned)K * 2u + chunk * 16u;
#pragma unroll
    for (int i = 0; i < TN; i++) wo[i] = (unsigned)min(n0 + srow + 32 * i, N - 1) * (unsigned)K * 2u + chunk * 16u;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    bf16_t* const a_dst = As + wave_u * 8 * LDS;     // the wave's 8 rows of every group of 32
    bf16_t* const b_dst = Bs + wave_u * 8 * LDS;
    auto fill = [&](int k0) {
        const char* xb = reinterpret_cast<const char*>(X) + (size_t)k0 * 2;
        const char* wb = reinterpret_cast<const char*>(W) + (size_t)k0 * 2;
#pragma unroll
        for (int i = 0; i < TM; i++)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xb + xo[i]),
                                             (__attribute__((address_space(3))) void*)(a_dst + 32 * i * LDS), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < TN; i++)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(wb + wo[i]),
                                             (__attribute__((address_space(3))) void*)(b_dst + 32 * i * LDS), 16, 0, 0);
    };
    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    auto frags = [&](int ks, Frag (&a)[TM], Frag (&b)[TN]) {
        const int kc = (((ks >> 3) + g) ^ (r & 7)) * 8;
#pragma unroll
        for (int i = 0; i < TM; i++) a[i].u = *reinterpret_cast<const uint4*>(As + (wm * 16 * TM + i * 16 + r) * LDS + kc);
#pragma unroll
        for (int j = 0; j < TN; j++) b[j].u = *reinterpret_cast<const uint4*>(Bs + (wn * 16 * TN + j * 16 + r) * LDS + kc);
    };
    auto mma = [&](Frag (&a)[TM], Frag (&b)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[j].v, a[i].v, acc[i][j], 0, 0, 0);
    };
    fill(k_begin);
    __builtin_amdgcn_s_waitcnt(0);                   // every counter at zero: the loads have reached LDS
    __syncthreads();
    for (int k0 = k_begin; k0 < k_end; k0 += BK) {
        Frag a0[TM], b0[TN], a1[TM], b1[TN];
        frags(0, a0, b0);
        frags(32, a1, b1);
        __builtin_amdgcn_s_waitcnt(0);               // the fragments are in registers ...
        __syncthreads();                             // ... everyone's: the buffer may be refilled
        if (k0 + BK < k_end) fill(k0 + BK);
        mma(a0, b0);
        mma(a1, b1);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
    }
    store_tile<EPI, TM, TN>(acc, Y, M, N, m0, n0, wm, wn, r, g, out_dtype, epi, units);
}

bool gemm_mfma_supports(const GemmArgs& a) {
    if (a.algo == 8 || a.algo == 9) return a.in_dtype == TP_BF16 && a.K % BK == 0 && (long)(a.M > a.N ? a.M : a.N) * a.K * 2 < (1L << 32);
    return a.in_dtype == TP_BF16 && a.K % 8 == 0;
}

// Tile of a product, in 16 x 16 tiles of a wave (the block is 2 x 2 waves), and its K slices.  Up to 64 rows:
// 64 x 64, the most blocks per byte of W.  Else 128 x 128 or 128 x 96 (three blocks a CU), by the loop that loads
// straight into LDS where K allows it; the register-staged loop also has 128 x 256 tiles (less LDS traffic per matrix
// instruction; two blocks fit a CU) for grids of at least four rounds of those 512 places (2B gate/up, register-staged:
// 930 against 790 TFLOP/s at 8192 rows, 700 against 790 at 2048).
struct Tile { int tm, tn, wm = 2; bool deep = false; };        // wm: waves along the rows of X (2 x 2 or 4 x 1)
struct Plan { Tile tile; int splits; bool direct = false; };

// K slices of a product of few rows, which is bound by reading W and wants every CU streaming.  From 17 rows on one
// block a CU: more slices cost their consumer more than they gain (a 2B decode step of 64 sequences takes 3.52 ms
// with 640 blocks, 3.34 with 256, 3.54 with 128).  Up to 16 rows the slices are small and the large matrices that
// come here want more blocks (a 27B step of 8 sequences: 13.6 ms with 640 blocks, 14.5 with 256).
static int small_tile_splits(const GemmArgs& a, long blocks) {
    if (blocks >= 512 || a.K < 512) return 1;
    int s = (int)tp_cdiv(a.M > 16 ? 256 : 640, blocks);
    if (s > a.K / 256) s = a.K / 256;
    if (s > 16) s = 16;
    return s < 1 ? 1 : s;
}

// The loop that loads straight into LDS takes whole k steps of 64 and 32-bit byte offsets of rows
static bool direct_ok(const GemmArgs& a) {
    return a.K % BK == 0 && (long)(a.M > a.N ? a.M : a.N) * a.K * 2 < (1L << 32);
}

// A grid that does not fill the chip's 256 CUs evenly runs as long as its fullest CU, and a CU holds three blocks at
// a time.  Microseconds per k step of the blocks a CU gets, with the loads straight into LDS: 1.43 for three blocks
// together, 1.17 for two, 1.0 for one alone (2B shapes: gate/up at 2,048 rows, nine blocks a CU, 36 steps: 155 us;
// qkv, two blocks: 42 us; o, 288 tiles: 37 us); a 128 x 96 block costs 0.8 of a 128 x 128 one.
static double direct_step_us(long blocks) {
    const long per_cu = tp_cdiv(blocks, 256), rest = per_cu % 3;
    return (double)(per_cu / 3) * 1.43 + (rest == 2 ? 1.17 : rest == 1 ? 1.0 : 0.0);
}

// (tile, K slices) of a product of many rows: the cheapest by the model above (register-staged loop, for a K that is
// no multiple of 64: the most blocks a CU gets x 0.64 us a step, fitted to the 2B down product at 2,048 rows), plus
// what writing and reading a further float32 slice of Y costs.
static Plan mid_tile_plan(const GemmArgs& a, bool may_slice) {
    const double step_us = 0.64, slice_us = (double)a.M * a.N * 8 / 4.0e6;
    const bool direct = direct_ok(a) && a.algo != 7;
    Plan best{{4, 4}, 1, direct};
    double best_cost = 1e30;
    for (int tn = 4; tn >= 3; tn--) {
        if (tn == 3 && a.epilogue == TP_EPI_GATED) continue;             // gate and up columns come in pairs of tiles
        const long tiles = (long)tp_cdiv(a.M, 128) * tp_cdiv(a.N, 32 * tn);
        for (int s = 1; s <= (may_slice ? 4 : 1); s++) {
            if (s > 1 && a.K / s < 512) break;
            const double k_steps = (double)tp_cdiv(tp_cdiv(a.K, s), BK);
            // a grid of at most one block a CU is faster by the register-staged loop (0.85 us a step against 1.0:
            // 128 x 96 tiles at 512 rows, 2B shapes: qkv 30.7 against 35.5 us, down 102 against 119)
            const bool d = direct && tiles * s > 256;
            const double per_step = d ? direct_step_us(tiles * s) : tiles * s <= 256 ? 0.85 : (double)tp_cdiv(tiles * s, 256) * step_us;
            const double cost = per_step * k_steps * (tn == 3 ? 0.8 : 1.0) + (s - 1) * slice_us;
            if (cost < best_cost * 0.97) { best_cost = cost; best = {{4, tn}, s, d}; }   // a tie stays with the earlier, plainer plan
        }
    }
    return best;
}

static Plan plan_of(const GemmArgs& a) {
    const bool may_slice = a.defer && a.epilogue == TP_EPI_NONE && (a.algo < 6 || a.algo == 11);
    if (a.algo == 10) return {{1, 2, 4, true}, 1};
    if (a.algo == 11) return {{2, 2, 2, true}, may_slice ? small_tile_splits(a, (long)tp_cdiv(a.M, 64) * tp_cdiv(a.N, 64)) : 1};
    if (a.algo == 6) return {{4, 8}, 1};
    if (a.algo == 7) return {{4, a.epilogue == TP_EPI_GATED ? 4 : 3}, 1};
    if (a.algo == 8) return {{4, 4}, 1, true};
    if (a.algo == 9) return {{4, a.epilogue == TP_EPI_GATED ? 4 : 3}, 1, true};
    // the logits of 64 rows: 250 us with 128 x 128, 275 with 64 x 64; up to 256 rows of a narrow product: 128 x 128
    // tiles would leave most CUs idle (down at 128 rows: 44 us on 72 blocks, against 15 us at 64 rows on 576 blocks
    // of 64 x 64; at 512 rows 128 x 128 wins again)
    if ((a.M <= 64 && !(a.M > 32 && a.N >= 32768)) || (a.M <= 256 && (long)tp_cdiv(a.M, 128) * tp_cdiv(a.N, 128) < 256)) {
        const long tiles = (long)tp_cdiv(a.M, 64) * tp_cdiv(a.N, 64);
        Tile t{2, 2};
        // Up to 32 rows what such a product waits for is W: with a second set of staging registers, so that a step's
        // loads are asked for a set earlier (the compiler still waits for all of them before a set's first use, so it
        // is less than two whole steps in flight), the long loops gain, those of a gated product
        // (never sliced) and of the slices of 17 rows and more (2B gate/up at 16 rows 27.6 -> 23.0 us, 27B at 8 rows
        // 141 -> 126, 9B qkv at 32 rows 21.1 -> 18.1); slices of a few steps (up to 16 rows) and 64 rows do not.
        // A gated product with about a block a CU in these tiles gains more from 64 x 32 tiles, twice the blocks with
        // the same bytes in flight each (2B gate/up at 8 to 24 rows: 27.7 -> 22.5 us; the 9B and 27B shapes do not).
        if (a.M <= 32 && (a.epilogue == TP_EPI_GATED || (may_slice && a.M > 16))) t.deep = true;
        if (a.M <= 32 && a.epilogue == TP_EPI_GATED && tiles <= 320) t = {1, 2, 4, true};
        return {t, may_slice ? small_tile_splits(a, tiles) : 1};
    }
    // register-staged loop only: 128 x 256 tiles from four rounds of their 512 places on
    if (!direct_ok(a) && (long)tp_cdiv(a.M, 128) * tp_cdiv(a.N, 256) >= 2048) return {{4, 8}, 1};
    return mid_tile_plan(a, may_slice);
}

// The plan with its slices as the launch makes them: a slice is a whole number of k steps, so fewer slices than were asked
// for may cover K (K 9216 in 16 slices: steps of 128 make 15 of 640), and the consumer must add exactly those written.
static Plan final_plan(const GemmArgs& a) {
    Plan p = plan_of(a);
    if (p.splits > 1) {
        const int kstep = p.tile.tm <= 2 ? SMALL_KS : BK;
        const int kps = tp_cdiv(tp_cdiv(a.K, p.splits), kstep) * kstep;
        p.splits = tp_cdiv(a.K, kps);
    }
    return p;
}

// K slices for products whose tiles alone do not fill the chip and whose consumer adds the slices (defer)
int gemm_mfma_splits(const GemmArgs& a) { return final_plan(a).splits; }

template <int EPI, int TM, int TN, int KS = BK, int WM = 2, bool DEEP = false>
static void mfma_launch(const GemmArgs& a, void* y, int out_dtype, int splits, int kps) {
    const int m_tiles = tp_cdiv(a.M, 16 * WM * TM), n_tiles = tp_cdiv(a.N, 16 * (4 / WM) * TN);
    dim3 grid((unsigned)(m_tiles * n_tiles), splits);
    const int xcd_panels = (long)m_tiles * n_tiles >= 1024 ? 1 : 0;
    if (TM > 2 && a.M >= 32 * TM && a.N >= 32 * TN)
        gemm_mfma_k<EPI, TM, TN, (TM > 2), KS><<<grid, 256, 0, a.stream>>>((const bf16_t*)a.x, (const bf16_t*)a.w, y, a.M, a.N, a.K, m_tiles,
                                                                      out_dtype, epi_constants(a), a.units, kps, xcd_panels);
    else
        gemm_mfma_k<EPI, TM, TN, false, KS, WM, DEEP><<<grid, 256, 0, a.stream>>>((const bf16_t*)a.x, (const bf16_t*)a.w, y, a.M, a.N, a.K, m_tiles,
                                                                       out_dtype, epi_constants(a), a.units, kps, xcd_panels);
}

template <int EPI>
static void mfma_launch_direct(const GemmArgs& a, Tile t, void* y, int out_dtype, int splits, int kps) {
    const int m_tiles = tp_cdiv(a.M, 128), n_tiles = tp_cdiv(a.N, 32 * t.tn);
    dim3 grid((unsigned)(m_tiles * n_tiles), splits);
    const int xcd_panels = (long)m_tiles * n_tiles >= 1024 ? 1 : 0;
    if (t.tn == 3) {
        if constexpr (EPI != TP_EPI_GATED)
            gemm_mfma_direct_k<EPI, 3><<<grid, 256, 0, a.stream>>>((const bf16_t*)a.x, (const bf16_t*)a.w, y, a.M, a.N, a.K, m_tiles,
                                                                   out_dtype, epi_constants(a), a.units, kps, xcd_panels);
    } else {
        gemm_mfma_direct_k<EPI, 4><<<grid, 256, 0, a.stream>>>((const bf16_t*)a.x, (const bf16_t*)a.w, y, a.M, a.N, a.K, m_tiles,
                                                               out_dtype, epi_constants(a), a.units, kps, xcd_panels);
    }
}

template <int EPI>
static void mfma_launch_tile(const GemmArgs& a, Tile t, void* y, int out_dtype, int splits, int kps) {
    if (t.wm == 4) mfma_launch<EPI, 1, 2, SMALL_KS, 4, true>(a, y, out_dtype, splits, kps);
    else if (t.tm == 2 && t.deep) mfma_launch<EPI, 2, 2, SMALL_KS, 2, true>(a, y, out_dtype, splits, kps);
    else if (t.tm == 2) mfma_launch<EPI, 2, 2, SMALL_KS>(a, y, out_dtype, splits, kps);
    else if (t.tn == 8) mfma_launch<EPI, 4, 8>(a, y, out_dtype, splits, kps);
    else if (t.tn == 3) {
        if constexpr (EPI != TP_EPI_GATED) mfma_launch<EPI, 4, 3>(a, y, out_dtype, splits, kps);
    } else mfma_launch<EPI, 4, 4>(a, y, out_dtype, splits, kps);
}

int gemm_mfma_launch(const GemmArgs& a) {
    TP_REQUIRE(gemm_mfma_supports(a), "tiled product: needs bf16 and K a multiple of 8 (K=%d)", a.K);
    TP_REQUIRE(((uintptr_t)a.x % 16 == 0) && ((uintptr_t)a.w % 16 == 0), "tiled product: operands must be 16-byte aligned");
    TP_REQUIRE(a.K < (1 << 22), "tiled product: K=%d exceeds the kernel's 32-bit offsets", a.K);
    TP_REQUIRE((long)tp_cdiv(a.M, 64) * tp_cdiv(a.N, 64) < (1L << 31), "tiled product: too many tiles for one launch (M=%d N=%d)", a.M, a.N);
    const Plan plan = final_plan(a);
    const Tile t = plan.tile;
    const int splits = plan.splits;
    if (splits > 1) {
        const size_t need = (size_t)splits * a.M * a.N * sizeof(float);
        TP_REQUIRE(a.workspace && a.workspace_bytes >= need, "tiled product: workspace of %zu bytes, %zu needed", a.workspace_bytes, need);
        const int kstep = t.tm <= 2 ? SMALL_KS : BK;
        const int kps = tp_cdiv(tp_cdiv(a.K, splits), kstep) * kstep;
        if (plan.direct) mfma_launch_direct<TP_EPI_NONE>(a, t, a.workspace, TP_F32, tp_cdiv(a.K, kps), kps);
        else mfma_launch_tile<TP_EPI_NONE>(a, t, a.workspace, TP_F32, tp_cdiv(a.K, kps), kps);
        return tp_check_launch("linear (tiled kernel, K slices)");
    }
    if (plan.direct) {
        if (a.epilogue == TP_EPI_GATED) mfma_launch_direct<TP_EPI_GATED>(a, t, a.y, a.out_dtype, 1, a.K);
        else if (a.epilogue == TP_EPI_SOFTCAP) mfma_launch_direct<TP_EPI_SOFTCAP>(a, t, a.y, a.out_dtype, 1, a.K);
        else mfma_launch_direct<TP_EPI_NONE>(a, t, a.y, a.out_dtype, 1, a.K);
        return tp_check_launch("linear (tiled kernel, loads into LDS)");
    }
    if (a.epilogue == TP_EPI_GATED) mfma_launch_tile<TP_EPI_GATED>(a, t, a.y, a.out_dtype, 1, a.K);
    else if (a.epilogue == TP_EPI_SOFTCAP) mfma_launch_tile<TP_EPI_SOFTCAP>(a, t, a.y, a.out_dtype, 1, a.K);
    else mfma_launch_tile<TP_EPI_NONE>(a, t, a.y, a.out_dtype, 1, a.K);
    return tp_check_launch("linear (tiled kernel)");
}
