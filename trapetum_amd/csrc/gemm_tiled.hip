// bf16 product for many rows, second kernel: 256 x 256 x 64 tiles, 8 waves, operands brought from global
// memory straight into LDS (no register staging) one K step ahead of the products.
//
// Block: 512 threads = 8 waves arranged 4 (along N) x 2 (along M); a wave owns 64 rows of W x 128 rows of X
// = 4 x 8 tiles of v_mfma_f32_16x16x32_bf16 (128 accumulator registers).  W rows are the A operand and X rows
// the B operand, so a lane ends up with 4 consecutive output columns of one output row (an 8-byte store), and
// with the gate and the up column of the same unit in two accumulators of the same lane.
// LDS holds two stages of (256 + 256) rows x 64 k.  Rows are 128 bytes, unpadded (the direct load writes a
// wave's 64 x 16 bytes contiguously); the 16-byte chunks of a row are stored at chunk ^ (row & 7) so that the
// 16 rows a fragment read touches spread over the banks.  The output goes through LDS once more, so that
// global stores are whole 128-byte rows.  Block ids are remapped so that the blocks one XCD receives (ids
// congruent modulo 8) work on neighbouring tiles and share W tiles in that XCD's L2.
// Needs K to be a multiple of 64 (a direct load cannot zero-fill); other shapes run on the first tiled kernel.
#include "gemm.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

namespace {
constexpr int TM = 256, TN = 256, TK = 64, NTH = 512;
constexpr int STAGE = (TM + TN) * TK;                 // elements per stage
constexpr int OLD = 64 + 8;                           // row stride of a wave's output tile in LDS (elements)
union Frag { uint4 u; bf16x8 v; };

__device__ __forceinline__ void load_to_lds(const bf16_t* src, bf16_t* dst_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)dst_wave_base, 16, 0, 0);
}
__device__ __forceinline__ bf16_t to_bf16(float f) { return f32_to_bf16(f); }
}

template <int EPI>
__global__ void __launch_bounds__(NTH)
gemm_tiled_k(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, void* __restrict__ Y,
             int M, int N, int K, int m_tiles, int out_dtype, float cap, int units) {
    extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wn = wave & 3, wm = wave >> 2;
    int L = blockIdx.x;
    if (gridDim.x % 8 == 0) L = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
    const int m0 = (L % m_tiles) * TM, n0 = (L / m_tiles) * TN;

    // ---- the wave's 8 direct loads per stage: j < 4 rows of W, j >= 4 rows of X; 8 rows of 128 bytes each ----
    const bf16_t* src[8];
    int dst[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int rb = (j & 3) * 8 + wave;                     // block of 8 rows within the operand's 256
        const int row = rb * 8 + (lane >> 3);
        const int gchunk = (lane & 7) ^ (lane >> 3);           // chunk of the row that lands at position lane & 7
        if (j < 4) {
            int n = n0 + row; n = n < N ? n : N - 1;
            src[j] = W + (size_t)n * K + gchunk * 8;
            dst[j] = rb * 8 * TK;
        } else {
            int m = m0 + row; m = m < M ? m : M - 1;
            src[j] = X + (size_t)m * K + gchunk * 8;
            dst[j] = TN * TK + rb * 8 * TK;
        }
    }
    auto issue = [&](int stage, int k0) {
#pragma unroll
        for (int j = 0; j < 8; j++) load_to_lds(src[j] + k0, lds + stage * STAGE + dst[j]);
    };

    f32x4 acc[4][8];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

    const int steps = K / TK;
    issue(0, 0);
    for (int s = 0; s < steps; s++) {
        if (s + 1 < steps) {
            issue((s + 1) & 1, (s + 1) * TK);
            __builtin_amdgcn_s_waitcnt(0xF78);                  // vmcnt(8): all but the 8 loads just issued have landed
        } else {
            __builtin_amdgcn_s_waitcnt(0xF70);                  // vmcnt(0)
        }
        __syncthreads();                                        // every wave's share of this stage is in LDS
        const bf16_t* ws = lds + (s & 1) * STAGE + (wn * 64) * TK;
        const bf16_t* xs = lds + (s & 1) * STAGE + TN * TK + (wm * 128) * TK;
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            const int chunk = ((ks * 4 + g) ^ (r & 7)) * 8;
            Frag a[4], b[8];
#pragma unroll
            for (int i = 0; i < 4; i++) a[i].u = *reinterpret_cast<const uint4*>(ws + (i * 16 + r) * TK + chunk);
#pragma unroll
            for (int j = 0; j < 8; j++) b[j].u = *reinterpret_cast<const uint4*>(xs + (j * 16 + r) * TK + chunk);
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 8; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i].v, b[j].v, acc[i][j], 0, 0, 0);
        }
        __syncthreads();                                        // the stage may be overwritten by the next issue
    }

    // ---- output: lane holds Y[m = .. + j*16 + r][n = .. + i*16 + g*4 + v] ----------------------------------------
    const int mw = m0 + wm * 128, nw = n0 + wn * 64;
    if (out_dtype == TP_F32) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int m = mw + j * 16 + r;
            if (m >= M) continue;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int n = nw + i * 16 + g * 4;
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    if (n + v >= N) continue;
                    float o = acc[i][j][v];
                    if (EPI == TP_EPI_SOFTCAP) o = softcap_f(o, cap);
                    ((float*)Y)[(size_t)m * N + n + v] = o;
                }
            }
        }
        return;
    }
    // bf16: through the wave's own 128 x 64 (or 128 x 32 units) tile in LDS, then whole rows to global memory
    bf16_t* ot = lds + wave * (128 * OLD);
    constexpr int COLS = EPI == TP_EPI_GATED ? 32 : 64;
#pragma unroll
    for (int j = 0; j < 8; j++) {
#pragma unroll
        for (int i = 0; i < 4; i += (EPI == TP_EPI_GATED ? 2 : 1)) {
            ushort4 pk;
            if (EPI == TP_EPI_GATED) {
                pk.x = to_bf16(gelu_tanh_f(acc[i][j][0]) * acc[i + 1][j][0]);
                pk.y = to_bf16(gelu_tanh_f(acc[i][j][1]) * acc[i + 1][j][1]);
                pk.z = to_bf16(gelu_tanh_f(acc[i][j][2]) * acc[i + 1][j][2]);
                pk.w = to_bf16(gelu_tanh_f(acc[i][j][3]) * acc[i + 1][j][3]);
                *reinterpret_cast<ushort4*>(ot + (j * 16 + r) * OLD + (i / 2) * 16 + g * 4) = pk;
            } else {
                pk.x = to_bf16(acc[i][j][0]); pk.y = to_bf16(acc[i][j][1]);
                pk.z = to_bf16(acc[i][j][2]); pk.w = to_bf16(acc[i][j][3]);
                *reinterpret_cast<ushort4*>(ot + (j * 16 + r) * OLD + i * 16 + g * 4) = pk;
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int out_cols = EPI == TP_EPI_GATED ? units : N;       // row length of Y
    const int cw = EPI == TP_EPI_GATED ? (nw >> 1) : nw;        // first output column of the wave
    constexpr int LPR = COLS / 8;                               // lanes per row (16 bytes each)
    constexpr int RPI = 64 / LPR;                               // rows per store instruction
    const int lr = lane / LPR, lc = (lane % LPR) * 8;
#pragma unroll
    for (int it = 0; it < 128 / RPI; it++) {
        const int ml = it * RPI + lr, m = mw + ml;
        if (m >= M) continue;
        const int col = cw + lc;
        bf16_t* yp = (bf16_t*)Y + (size_t)m * out_cols + col;
        if (col + 8 <= out_cols && (out_cols % 8) == 0) {
            *reinterpret_cast<uint4*>(yp) = *reinterpret_cast<const uint4*>(ot + ml * OLD + lc);
        } else {
            for (int e = 0; e < 8; e++)
                if (col + e < out_cols) yp[e] = ot[ml * OLD + lc + e];
        }
    }
}

bool gemm_tiled_supports(const GemmArgs& a) {
    return a.in_dtype == TP_BF16 && a.K % TK == 0 && a.K >= TK && a.M > 64 &&
           !(a.epilogue == TP_EPI_GATED && a.out_dtype == TP_F32);
}

template <int EPI>
static int tiled_launch(const GemmArgs& a, int m_tiles, long blocks, size_t smem) {
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_tiled_k<EPI>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return tp_fail("tiled product: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
        configured = true;
    }
    gemm_tiled_k<EPI><<<(unsigned)blocks, NTH, smem, a.stream>>>((const bf16_t*)a.x, (const bf16_t*)a.w, a.y, a.M, a.N, a.K,
                                                                  m_tiles, a.out_dtype, a.cap, a.units);
    return tp_check_launch("linear (tiled kernel, direct loads)");
}

int gemm_tiled_launch(const GemmArgs& a) {
    TP_REQUIRE(gemm_tiled_supports(a), "tiled product (direct loads): needs bf16, more than 64 rows and K a multiple of 64 (M=%d K=%d)", a.M, a.K);
    TP_REQUIRE(((uintptr_t)a.x % 16 == 0) && ((uintptr_t)a.w % 16 == 0), "tiled product: operands must be 16-byte aligned");
    const int m_tiles = tp_cdiv(a.M, TM), n_tiles = tp_cdiv(a.N, TN);
    const long blocks = (long)m_tiles * n_tiles;
    TP_REQUIRE(blocks < (1L << 31), "tiled product: %ld tiles are too many for one launch", blocks);
    size_t smem = (size_t)2 * STAGE * sizeof(bf16_t);
    const size_t out_bytes = (size_t)8 * 128 * OLD * sizeof(bf16_t);
    if (out_bytes > smem) smem = out_bytes;
    if (a.epilogue == TP_EPI_GATED) return tiled_launch<TP_EPI_GATED>(a, m_tiles, blocks, smem);
    if (a.epilogue == TP_EPI_SOFTCAP) return tiled_launch<TP_EPI_SOFTCAP>(a, m_tiles, blocks, smem);
    return tiled_launch<TP_EPI_NONE>(a, m_tiles, blocks, smem);
}
