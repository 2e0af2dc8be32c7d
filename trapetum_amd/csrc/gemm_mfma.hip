// bf16 product for many rows (prefill): LDS-tiled, on the matrix cores, fp32 accumulation.
//
// Block: 256 threads = 4 waves in a 2 x 2 arrangement over a 128 x 128 tile of Y; each wave owns
// 64 x 64 = 4 x 4 tiles of v_mfma_f32_16x16x32_bf16.  X rows are the A operand and W rows the B operand
// (both are contiguous along k, which is what the instruction wants per lane), so a lane ends up with
// 4 consecutive rows of one output column, and with the gate and the up column of the same unit in two
// accumulators of the same lane (the packed gate/up matrix alternates 16 gate rows and 16 up rows).
// K is walked in steps of 64 through one LDS buffer; the next step's global loads are issued before the
// current step's products and written to LDS after them.  The 16-byte chunks of an LDS row are stored at
// chunk ^ (row & 7), so that the 16 rows a fragment read touches spread over the banks (measured: bank
// conflicts fall from a third of the LDS cycles with padded rows to a few per cent).
// Consecutive block ids walk the M tiles of one N tile, so blocks in flight together share W tiles.
#include "gemm.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

namespace {
constexpr int BM = 128, BN = 128, BK = 64, LDS = BK;          // LDS row stride in elements (128 bytes, unpadded)
union Frag { uint4 u; bf16x8 v; };
}

template <int EPI>
__global__ void __launch_bounds__(256)
gemm_mfma_k(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, void* __restrict__ Y,
            int M, int N, int K, int m_tiles, int out_dtype, float cap, int units, int k_per_split) {
    __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDS];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * LDS];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = (blockIdx.x % m_tiles) * BM, n0 = (blockIdx.x / m_tiles) * BN;
    // a K slice per blockIdx.y: slices go to Y as float32 [slices, M, N] for the consumer to add in slice order
    const int k_begin = blockIdx.y * k_per_split;
    const int k_end = min(K, k_begin + k_per_split);
    if (gridDim.y > 1) Y = (float*)Y + (size_t)blockIdx.y * M * N;

    // global -> register staging: 4 chunks of 16 bytes per thread and operand; chunk c: row c / 8, k chunk c % 8
    uint4 ra[4], rb[4];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int c = tid + i * 256, row = c >> 3, kc = (c & 7) * 8;
            const int k = k0 + kc;
            const int m = m0 + row, n = n0 + row;
            ra[i] = (m < M && k < k_end) ? *reinterpret_cast<const uint4*>(X + (size_t)m * K + k) : make_uint4(0, 0, 0, 0);
            rb[i] = (n < N && k < k_end) ? *reinterpret_cast<const uint4*>(W + (size_t)n * K + k) : make_uint4(0, 0, 0, 0);
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int c = tid + i * 256, row = c >> 3, kc = ((c & 7) ^ (row & 7)) * 8;    // chunk j of a row sits at j ^ (row & 7)
            *reinterpret_cast<uint4*>(As + row * LDS + kc) = ra[i];
            *reinterpret_cast<uint4*>(Bs + row * LDS + kc) = rb[i];
        }
    };

    f32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

    fetch(k_begin);
    for (int k0 = k_begin; k0 < k_end; k0 += BK) {
        __syncthreads();                       // everyone is done reading the previous tile
        stage();
        __syncthreads();
        if (k0 + BK < k_end) fetch(k0 + BK);
#pragma unroll
        for (int ks = 0; ks < BK; ks += 32) {
            Frag a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int kc = (((ks >> 3) + g) ^ (r & 7)) * 8;
                a[i].u = *reinterpret_cast<const uint4*>(As + (wm * 64 + i * 16 + r) * LDS + kc);
                b[i].u = *reinterpret_cast<const uint4*>(Bs + (wn * 64 + i * 16 + r) * LDS + kc);
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i].v, b[j].v, acc[i][j], 0, 0, 0);
        }
    }

    // lane holds Y[m = .. + g*4 + v][n = .. + r]
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int m = m0 + wm * 64 + i * 16 + g * 4 + v;
            if (m >= M) continue;
            if (EPI == TP_EPI_GATED) {
#pragma unroll
                for (int j = 0; j < 4; j += 2) {
                    const int unit = ((n0 + wn * 64 + j * 16) >> 1) + r;
                    if (unit < units) {
                        const float o = gelu_tanh_f(acc[i][j][v]) * acc[i][j + 1][v];
                        if (out_dtype == TP_F32) ((float*)Y)[(size_t)m * units + unit] = o;
                        else ((bf16_t*)Y)[(size_t)m * units + unit] = f32_to_bf16(o);
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int n = n0 + wn * 64 + j * 16 + r;
                    if (n >= N) continue;
                    float o = acc[i][j][v];
                    if (EPI == TP_EPI_SOFTCAP) o = softcap_f(o, cap);
                    if (out_dtype == TP_F32) ((float*)Y)[(size_t)m * N + n] = o;
                    else ((bf16_t*)Y)[(size_t)m * N + n] = f32_to_bf16(o);
                }
            }
        }
    }
}

bool gemm_mfma_supports(const GemmArgs& a) {
    return a.in_dtype == TP_BF16 && a.K % 8 == 0;
}

// K slices for products whose tiles alone do not fill the chip and whose consumer adds the slices (defer)
int gemm_mfma_splits(const GemmArgs& a) {
    if (!a.defer || a.epilogue != TP_EPI_NONE) return 1;
    const long blocks = (long)tp_cdiv(a.M, BM) * tp_cdiv(a.N, BN);
    if (blocks >= 448 || a.K < 1024) return 1;          // measured at 288 tiles: the slices win back a fifth
    int s = (int)(640 / blocks);
    if (s > a.K / 512) s = a.K / 512;
    if (s > 4) s = 4;
    return s < 1 ? 1 : s;
}

int gemm_mfma_launch(const GemmArgs& a) {
    TP_REQUIRE(gemm_mfma_supports(a), "tiled product: needs bf16 and K a multiple of 8 (K=%d)", a.K);
    TP_REQUIRE(((uintptr_t)a.x % 16 == 0) && ((uintptr_t)a.w % 16 == 0), "tiled product: operands must be 16-byte aligned");
    const int m_tiles = tp_cdiv(a.M, BM), n_tiles = tp_cdiv(a.N, BN);
    const long blocks = (long)m_tiles * n_tiles;
    TP_REQUIRE(blocks < (1L << 31), "tiled product: %ld tiles are too many for one launch", blocks);
    const bf16_t* x = (const bf16_t*)a.x;
    const bf16_t* w = (const bf16_t*)a.w;
    const int splits = gemm_mfma_splits(a);
    if (splits > 1) {
        const size_t need = (size_t)splits * a.M * a.N * sizeof(float);
        TP_REQUIRE(a.workspace && a.workspace_bytes >= need, "tiled product: workspace of %zu bytes, %zu needed", a.workspace_bytes, need);
        const int kps = tp_cdiv(tp_cdiv(a.K, splits), BK) * BK;
        dim3 grid((unsigned)blocks, tp_cdiv(a.K, kps));
        gemm_mfma_k<TP_EPI_NONE><<<grid, 256, 0, a.stream>>>(x, w, a.workspace, a.M, a.N, a.K, m_tiles, TP_F32, 0.f, 0, kps);
        return tp_check_launch("linear (tiled kernel, K slices)");
    }
    if (a.epilogue == TP_EPI_GATED)
        gemm_mfma_k<TP_EPI_GATED><<<(unsigned)blocks, 256, 0, a.stream>>>(x, w, a.y, a.M, a.N, a.K, m_tiles, a.out_dtype, a.cap, a.units, a.K);
    else if (a.epilogue == TP_EPI_SOFTCAP)
        gemm_mfma_k<TP_EPI_SOFTCAP><<<(unsigned)blocks, 256, 0, a.stream>>>(x, w, a.y, a.M, a.N, a.K, m_tiles, a.out_dtype, a.cap, a.units, a.K);
    else
        gemm_mfma_k<TP_EPI_NONE><<<(unsigned)blocks, 256, 0, a.stream>>>(x, w, a.y, a.M, a.N, a.K, m_tiles, a.out_dtype, a.cap, a.units, a.K);
    return tp_check_launch("linear (tiled kernel)");
}
