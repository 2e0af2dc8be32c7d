// Entry points of the matrix products and the plain tiled kernel.
//
// The plain kernel is the whole of the float32 path (no matrix-core mode, every output element summed
// over k in index order whatever the batch is) and the fallback of the bf16 path for shapes the
// matrix-core kernels refuse.  The reference's products are 4-bit codebook GEMVs
// (runtime/cuda/codebook_gemv.cu:86-114); its only dense one is gemv_fp16_warp_k (cu:496-517).
#include "gemm.h"

// A block of 16 x 16 threads owns a tile of 16 R x 16 R outputs, R x R per thread, and walks K in steps of BK
// through LDS.  Every output is one chain acc = fma(x, w, acc) over k = 0, 1, 2, ...: the same bits for every R,
// BK and batch.  R = 4 for many rows; R = 1 (sixteen times the blocks, whole 256-byte pieces of a row per load)
// for the few rows of a decode step, where a narrow product would otherwise run on a few dozen blocks.
template <typename TI, typename TO, int R, int BK>
__global__ void __launch_bounds__(256)
gemm_simple_k(const TI* __restrict__ X, const TI* __restrict__ W, TO* __restrict__ Y, int M, int N, int K, float cap) {
    constexpr int T = 16 * R;
    __shared__ float xs[BK][T + 1];
    __shared__ float ws[BK][T + 1];
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * T, n0 = blockIdx.x * T;
    float acc[R][R] = {};
    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int i = 0; i < T * BK / 256; i++) {
            const int idx = tid + i * 256, r = idx / BK, kk = idx % BK;
            const int k = k0 + kk;
            xs[kk][r] = (m0 + r < M && k < K) ? ld_f32(X + (size_t)(m0 + r) * K + k) : 0.f;
            ws[kk][r] = (n0 + r < N && k < K) ? ld_f32(W + (size_t)(n0 + r) * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll 16
        for (int kk = 0; kk < BK; kk++) {
            float a[R], b[R];
#pragma unroll
            for (int i = 0; i < R; i++) { a[i] = xs[kk][ty * R + i]; b[i] = ws[kk][tx * R + i]; }
#pragma unroll
            for (int i = 0; i < R; i++)
#pragma unroll
                for (int j = 0; j < R; j++) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < R; i++) {
        const int m = m0 + ty * R + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < R; j++) {
            const int n = n0 + tx * R + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (cap > 0.f) v = softcap_f(v, cap);
            st_f32(Y + (size_t)m * N + n, v);
        }
    }
}

extern "C" int tp_gated_act(const float* y, void* out, int dtype, int M, int I, int act, void* stream);

template <typename TI>
static int simple_typed(const GemmArgs& a, void* y, int out_dtype, float cap) {
    if (a.M <= 16) {
        dim3 grid(tp_cdiv(a.N, 16), 1);
        if (out_dtype == TP_F32)
            gemm_simple_k<TI, float, 1, 64><<<grid, 256, 0, a.stream>>>((const TI*)a.x, (const TI*)a.w, (float*)y, a.M, a.N, a.K, cap);
        else
            gemm_simple_k<TI, bf16_t, 1, 64><<<grid, 256, 0, a.stream>>>((const TI*)a.x, (const TI*)a.w, (bf16_t*)y, a.M, a.N, a.K, cap);
        return tp_check_launch("linear (plain kernel, few rows)");
    }
    dim3 grid(tp_cdiv(a.N, 64), tp_cdiv(a.M, 64));
    if (out_dtype == TP_F32)
        gemm_simple_k<TI, float, 4, 16><<<grid, 256, 0, a.stream>>>((const TI*)a.x, (const TI*)a.w, (float*)y, a.M, a.N, a.K, cap);
    else
        gemm_simple_k<TI, bf16_t, 4, 16><<<grid, 256, 0, a.stream>>>((const TI*)a.x, (const TI*)a.w, (bf16_t*)y, a.M, a.N, a.K, cap);
    return tp_check_launch("linear (plain kernel)");
}

int gemm_simple_launch(const GemmArgs& a) {
    void* y = a.y;
    int out_dtype = a.out_dtype;
    if (a.epilogue == TP_EPI_GATED) {
        TP_REQUIRE(a.workspace && a.workspace_bytes >= (size_t)a.M * a.N * 4, "gated product: workspace of %zu bytes is too small", a.workspace_bytes);
        y = a.workspace;
        out_dtype = TP_F32;
    }
    const float cap = a.epilogue == TP_EPI_SOFTCAP ? a.cap : 0.f;
    int rc = a.in_dtype == TP_BF16 ? simple_typed<bf16_t>(a, y, out_dtype, cap) : simple_typed<float>(a, y, out_dtype, cap);
    if (rc) return rc;
    if (a.epilogue == TP_EPI_GATED) return tp_gated_act((const float*)y, a.y, a.out_dtype, a.M, a.units, a.act, a.stream);
    return 0;
}

static int check_args(const GemmArgs& a) {
    TP_REQUIRE(a.M > 0 && a.N > 0 && a.K > 0, "linear: empty shape M=%d N=%d K=%d", a.M, a.N, a.K);
    TP_REQUIRE(a.in_dtype == TP_F32 || a.in_dtype == TP_BF16, "linear: unknown input dtype %d", a.in_dtype);
    TP_REQUIRE(a.out_dtype == TP_F32 || a.out_dtype == TP_BF16, "linear: unknown output dtype %d", a.out_dtype);
    TP_REQUIRE(!(a.in_dtype == TP_F32 && a.out_dtype == TP_BF16), "linear: float32 rows give float32 output");
    TP_REQUIRE(a.epilogue != TP_EPI_SOFTCAP || a.cap > 0.f, "linear: a soft cap must be positive");
    TP_REQUIRE(!a.defer || a.epilogue == TP_EPI_NONE, "linear: K slices can be left to the consumer only without an epilogue (found %d)", a.epilogue);
    if (a.epilogue == TP_EPI_GATED) {
        const int padded = 2 * ((a.units + 15) / 16) * 16;
        TP_REQUIRE(a.units > 0 && a.N == padded, "gated product: %d units need a packed matrix of %d rows, found %d", a.units, padded, a.N);
        float c1, c3;
        TP_REQUIRE(tp_gate_constants(a.act, &c1, &c3), "gated product: activation %d is neither gelu-tanh (%d) nor SiLU (%d)", a.act, TP_ACT_GELU_TANH, TP_ACT_SILU);
    }
    return 0;
}

// algo: 0 = choose, 1 = plain, 2 = skinny matrix-core, 3 = tiled matrix-core (6: with its wide tile, 7: with its 128 x 96 tile,
// 8, 9: with its loop that loads straight into LDS, 128 x 128 and 128 x 96; 10, 11: its 64 x 32 and 64 x 64 tiles with two k
// steps asked for ahead), 4 = multiply-adds for one or two rows, 5 = matrix-core kernel for up to eight rows
static int pick(const GemmArgs& a, int algo) {
    if (algo == 1) return 1;
    if (algo == 4) return gemv_supports(a) ? 4 : -4;
    if (algo == 5) return gemm_rows8_supports(a) ? 5 : -5;
    if (algo == 2) return gemm_skinny_supports(a) ? 2 : -2;
    if (algo == 3 || (algo >= 6 && algo <= 11)) return gemm_mfma_supports(a) ? 3 : -3;
    // Up to 64 rows both matrix-core kernels stream W once; which is faster was measured on MI355X at the 2B shapes
    // (cold weights, microseconds, skinny / tiled with 64 x 64 tiles and k steps of 128):
    //   logits  N 256000            8 rows 277 / 222
    //   down    N 2304  K 9216      8 rows 15.8 / 11.3   32 rows 20.1 / 12.0   64 rows 26.3 / 13.5   (K slices left to the consumer)
    //   qkv     N 4096  K 2304      8 rows  8.0 /  7.1   32 rows 11.7 /  7.5   64 rows 13.5 /  8.5   (K slices)
    //   o       N 2304  K 2048      8 rows  5.2 /  5.5   32 rows  7.7 /  6.0   64 rows 13.3 /  6.7   (K slices)
    //   gate/up N 18432 K 2304      8 rows 26.9 / 24.2   32 rows 40.7 / 24.7   64 rows 48.5 / 26.5   (no slices: gated)
    if (gemv_supports(a)) return 4;          // one or two rows: 2B gate/up 16.8 against 22.6 us on the skinny kernel
    // Three to eight rows: the kernel whose blocks read 8 rows of W in one go, where it was measured faster than the
    // choice below (microseconds from a replayed graph, cold weights, that choice / this kernel / a kernel that only reads):
    //   2B  gate/up 24.1 / 21.7 / 15.2   down 14.5 / 11.5 / 9.1   qkv 7.1 / 6.3 / 4.9   o 5.0 / 5.2 / 4.2   logits 209 / 253 / 204
    //   9B  gate/up 43.2 / 45.6 / 36.1   down 22.0 / 24.5 / 18.6  qkv 13.5 / 15.1 / 12.1  o 10.0 / 9.2 / 7.6
    //   27B gate/up 141 / 136 / 116      down 72.4 / 76.7 / 58.2  qkv 16.8 / 19.9 / 14.9  o 14.5 / 10.8 / 8.3   logits 407 / 462 / 414
    // at 8 rows; at 3 and 4 rows, where the choice below is the skinny kernel, 2B logits 250 / 228, 9B gate/up 49.3 / 41.8,
    // 27B gate/up 142 / 127, 27B qkv 16.9 / 19.4.  A slice of K beyond 2,304 takes the kernel a second round of loads.
    // A decode step of 8 sequences at the 2B sizes: 2.30 -> 2.00 ms.
    // The bounds below are what those measurements have in common, in the kernels' own terms:
    //   ONE_ROUND_K  the K a block of the 8-row kernel reads in one round of loads (TP_R8_MAX_STEPS steps of 64 k by four
    //                waves): beyond it the kernel loops, and a slice of K left to the consumer keeps it within one round;
    //   WIDE_N       from here on a product is the logits' kind: so many rows of W that the tiled kernel's 64 x 64 tiles
    //                fill every CU several times over (512 tiles = two a CU) and its larger k steps win;
    //   LARGE_NK     elements of W from which the tiled kernel's streaming wins at 8 rows and more (the 27B matrices and
    //                every gated product: 340 MB, 93 -> 74 us), measured between 21 M (2B down: the 8-row kernel wins)
    //                and 42 M (2B gate/up: the tiled kernel wins);
    //   R8_SLICED_NK elements of W up to which the 8-row kernel, its K in slices for the consumer, beat the tiled kernel
    //                in a whole step (all the 2B and 9B products but the 9B feed-forward; the 27B ones lose).
    constexpr int ONE_ROUND_K = TP_R8_MAX_STEPS * 256, WIDE_N = 64 * 512;
    constexpr long LARGE_NK = 24000000, R8_SLICED_NK = 32000000;
    if (a.M <= 8 && gemm_rows8_supports(a)) {
        const long nk = (long)a.N * a.K;
        if (a.defer && a.epilogue == TP_EPI_NONE) {
            if (nk <= R8_SLICED_NK) return 5;     // (2B o alone is no faster, 5.0 / 5.2, but a step of 8 sequences is: 2.001 -> 1.988 ms)
        } else if (a.M < 8) {
            if (a.epilogue == TP_EPI_GATED || a.K <= ONE_ROUND_K || a.N >= WIDE_N) return 5;
        } else if (a.K <= ONE_ROUND_K && a.N < WIDE_N) {
            return 5;
        }
    }
    if (gemm_mfma_supports(a)) {
        const bool sliced = a.defer && a.epilogue == TP_EPI_NONE;
        // (at 8 rows the tiled kernel's lead on qkv and down is lost again in their consumers, which then add 9 and 16
        // slices instead of 2 and 4; a single sequence is faster on the skinny kernel throughout)
        if (a.M >= 8 && (a.epilogue == TP_EPI_GATED || (long)a.N * a.K >= LARGE_NK)) return 3;
        if (a.M >= 8 && a.N >= WIDE_N) return 3;
        // from 9 rows on the tiled kernel wins every product of a layer against the skinny one (2B, 16 rows, cold
        // weights: qkv 6.4 / 8.0 us, o 5.1 / 5.3, down 11.5 / 18.6; a step of 16 sequences 2.47 -> 2.32 ms)
        if (a.M > 8 && (sliced || a.N >= 8192)) return 3;
    }
    if (gemm_skinny_supports(a)) return 2;
    if (gemm_mfma_supports(a)) return 3;
    return 1;
}

// bytes of workspace a product needs; with defer, a positive multiple of M * N * 4 above one slice means the
// product comes back as that many K slices
extern "C" long tp_linear_workspace_bytes(int in_dtype, int out_dtype, int M, int N, int K, int epilogue, int units,
                                          int defer, int algo) {
    GemmArgs a{nullptr, nullptr, nullptr, in_dtype, out_dtype, M, N, K, epilogue, 1.f, units, 0, nullptr, 0, defer, algo, nullptr};
    const int p = pick(a, algo);
    if (p == 2) return (long)gemm_skinny_workspace(a);
    if (p == 4) return (long)gemv_workspace(a);
    if (p == 5) return (long)gemm_rows8_workspace(a);
    if (p == 3) { const int s = gemm_mfma_splits(a); return s > 1 ? (long)s * M * N * 4 : 0; }
    if (p == 1 && epilogue == TP_EPI_GATED) return (long)M * N * 4;
    return 0;
}

extern "C" int tp_linear(const void* x, const void* w, void* y, int in_dtype, int out_dtype, int M, int N, int K,
                         int epilogue, float cap, int units, int act, void* workspace, long workspace_bytes, int defer,
                         int algo, void* stream) {
    GemmArgs a{x, w, y, in_dtype, out_dtype, M, N, K, epilogue, cap, units, act, workspace, (size_t)workspace_bytes, defer,
               algo, (hipStream_t)stream};
    if (int rc = check_args(a)) return rc;
    const int p = pick(a, algo);
    TP_REQUIRE(p > 0, "linear: the requested kernel (%d) does not take M=%d N=%d K=%d dtype %d", algo, M, N, K, in_dtype);
    if (p == 2) return gemm_skinny_launch(a);
    if (p == 4) return gemv_launch(a);
    if (p == 5) return gemm_rows8_launch(a);
    if (p == 3) return gemm_mfma_launch(a);
    return gemm_simple_launch(a);
}
