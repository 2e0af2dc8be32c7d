// bf16 product for one or two rows (a decode step of one or two sequences) by plain multiply-adds.
//
// With so few rows the matrix cores have nothing to gain, and their operand layout costs: a fragment load of
// X for every fragment of W.  Here a wave owns two rows of W over the block's K slice; a lane keeps the X values
// that belong to its k positions in registers for the whole kernel (chunk c of a lane: 8 elements at
// (c * 64 + lane) * 8), so that only W streams, a contiguous kilobyte per wave and load.  A lane's products are
// summed in k order, the 64 lanes by the butterfly of wave_sum: an order that depends on K alone.  K slices (K
// beyond what the registers take) go to the workspace as float32 [slices, M, N] for the consumer to add in slice
// order, like the other products'.  Measured on MI355X at the 2B shapes, one row, cold weights, against the
// skinny matrix-core kernel: gate/up 16.8 / 22.6 us, down 10.4 / 12.4, qkv 5.4 / 6.8, o 4.3 / 5.0.
// The reference's dense product of one row is gemv_fp16_warp_k (runtime/cuda/codebook_gemv.cu:496-517): a warp a
// row, 16-byte loads, a shuffle reduction.
#include "gemm.h"

namespace {
constexpr int GV_ROWS = 2;                       // rows of W a wave takes (for a gated product: a unit's gate and up row)
constexpr int GV_MAX_CHUNKS = 10;                // chunks of 512 k a lane can hold: K slices of at most 5,120

__device__ __forceinline__ float lo_f32(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float hi_f32(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }
}

// MR: rows of X (1 or 2); NC: chunks of 512 k per lane
template <int MR, int NC>
__global__ void __launch_bounds__(256)
gemv_k(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, void* __restrict__ Y, float* __restrict__ part,
       int M, int N, int K, int k_per_split, int n_splits, int out_dtype, int epilogue, float2 epi, int units) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int kbeg = blockIdx.y * k_per_split, klen = min(K, kbeg + k_per_split) - kbeg;
    // a chunk past the slice reads the slice's first elements (loads stay unconditional) against X values of zero
    uint4 xr[MR][NC];
    int kof[NC];
#pragma unroll
    for (int c = 0; c < NC; c++) {
        const int k = (c * 64 + lane) * 8;
        const bool ok = k < klen;
        kof[c] = kbeg + (ok ? k : 0);
#pragma unroll
        for (int m = 0; m < MR; m++) {
            uint4 t = *reinterpret_cast<const uint4*>(X + (size_t)(m < M ? m : 0) * K + kof[c]);
            if (!(ok && m < M)) t = make_uint4(0, 0, 0, 0);
            xr[m][c] = t;
        }
    }
    // the wave's two rows: neighbours, or the gate row and the up row of one unit (the packed matrix alternates 16
    // gate rows and the 16 up rows of the same units)
    const int item = blockIdx.x * 4 + wave;
    int row[GV_ROWS];
    if (epilogue == TP_EPI_GATED) {
        row[0] = (item >> 4) * 32 + (item & 15);
        row[1] = row[0] + 16;
    } else {
        row[0] = item * 2;
        row[1] = item * 2 + 1;
    }
    uint4 w[GV_ROWS][NC];
#pragma unroll
    for (int j = 0; j < GV_ROWS; j++) {
        const bf16_t* wr = W + (size_t)min(row[j], N - 1) * K;
#pragma unroll
        for (int c = 0; c < NC; c++) w[j][c] = *reinterpret_cast<const uint4*>(wr + kof[c]);
    }
    float acc[GV_ROWS][MR];
#pragma unroll
    for (int j = 0; j < GV_ROWS; j++) {
#pragma unroll
        for (int m = 0; m < MR; m++) acc[j][m] = 0.f;
#pragma unroll
        for (int c = 0; c < NC; c++) {
            const uint32_t wv[4] = {w[j][c].x, w[j][c].y, w[j][c].z, w[j][c].w};
#pragma unroll
            for (int m = 0; m < MR; m++) {
                const uint32_t xv[4] = {xr[m][c].x, xr[m][c].y, xr[m][c].z, xr[m][c].w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    acc[j][m] = fmaf(lo_f32(wv[e]), lo_f32(xv[e]), acc[j][m]);
                    acc[j][m] = fmaf(hi_f32(wv[e]), hi_f32(xv[e]), acc[j][m]);
                }
            }
        }
#pragma unroll
        for (int m = 0; m < MR; m++) acc[j][m] = wave_sum(acc[j][m]);
    }
    if (lane != 0) return;
#pragma unroll
    for (int m = 0; m < MR; m++) {
        if (m >= M) break;
        if (n_splits > 1) {
#pragma unroll
            for (int j = 0; j < GV_ROWS; j++)
                if (row[j] < N) part[((size_t)blockIdx.y * M + m) * N + row[j]] = acc[j][m];
        } else if (epilogue == TP_EPI_GATED) {
            if (item < units) {
                const float o = gate_act_fast(acc[0][m], epi) * acc[1][m];
                if (out_dtype == TP_F32) ((float*)Y)[(size_t)m * units + item] = o;
                else ((bf16_t*)Y)[(size_t)m * units + item] = f32_to_bf16(o);
            }
        } else {
#pragma unroll
            for (int j = 0; j < GV_ROWS; j++) {
                if (row[j] >= N) continue;
                float o = acc[j][m];
                if (epilogue == TP_EPI_SOFTCAP) o = softcap_f(o, epi.x);
                if (out_dtype == TP_F32) ((float*)Y)[(size_t)m * N + row[j]] = o;
                else ((bf16_t*)Y)[(size_t)m * N + row[j]] = f32_to_bf16(o);
            }
        }
    }
}

// K slices: as few as the registers allow, of equal length (a multiple of 8)
static void gemv_plan(const GemmArgs& a, int& splits, int& kps) {
    splits = tp_cdiv(a.K, GV_MAX_CHUNKS * 512 / 2);          // slices of at most 2,560: five chunks, the fastest form
    if (a.epilogue != TP_EPI_NONE || !a.defer) splits = 1;   // nobody would add the slices
    kps = tp_cdiv(tp_cdiv(a.K, splits), 8) * 8;
    splits = tp_cdiv(a.K, kps);
}

bool gemv_supports(const GemmArgs& a) {
    if (!(a.in_dtype == TP_BF16 && a.M <= 2 && a.K % 8 == 0)) return false;
    int splits, kps;
    gemv_plan(a, splits, kps);
    return kps <= GV_MAX_CHUNKS * 512;
}

size_t gemv_workspace(const GemmArgs& a) {
    int splits, kps;
    gemv_plan(a, splits, kps);
    return splits > 1 ? (size_t)splits * a.M * a.N * sizeof(float) : 0;
}

template <int MR, int NC>
static void gemv_launch_nc(const GemmArgs& a, dim3 grid, float* part, int kps, int splits) {
    gemv_k<MR, NC><<<grid, 256, 0, a.stream>>>((const bf16_t*)a.x, (const bf16_t*)a.w, a.y, part, a.M, a.N, a.K, kps, splits,
                                              a.out_dtype, a.epilogue, epi_constants(a), a.units);
}

template <int MR>
static void gemv_launch_mr(const GemmArgs& a, dim3 grid, float* part, int kps, int splits) {
    const int nc = tp_cdiv(kps, 512);
    if (nc <= 2) gemv_launch_nc<MR, 2>(a, grid, part, kps, splits);
    else if (nc <= 3) gemv_launch_nc<MR, 3>(a, grid, part, kps, splits);
    else if (nc <= 4) gemv_launch_nc<MR, 4>(a, grid, part, kps, splits);
    else if (nc <= 5) gemv_launch_nc<MR, 5>(a, grid, part, kps, splits);
    else if (nc <= 7) gemv_launch_nc<MR, 7>(a, grid, part, kps, splits);
    else gemv_launch_nc<MR, GV_MAX_CHUNKS>(a, grid, part, kps, splits);
}

int gemv_launch(const GemmArgs& a) {
    TP_REQUIRE(gemv_supports(a), "product of few rows: needs bf16, at most 2 rows, K a multiple of 8 and (unsliced) at most %d (M=%d K=%d)",
               GV_MAX_CHUNKS * 512, a.M, a.K);
    TP_REQUIRE(((uintptr_t)a.x % 16 == 0) && ((uintptr_t)a.w % 16 == 0), "product of few rows: operands must be 16-byte aligned");
    int splits, kps;
    gemv_plan(a, splits, kps);
    float* part = nullptr;
    if (splits > 1) {
        const size_t need = (size_t)splits * a.M * a.N * sizeof(float);
        TP_REQUIRE(a.workspace && a.workspace_bytes >= need, "product of few rows: workspace of %zu bytes, %zu needed", a.workspace_bytes, need);
        part = (float*)a.workspace;
    }
    // a block's four waves take four items: pairs of rows, or units of a gated product (padded to whole tiles of 16)
    const long items = a.epilogue == TP_EPI_GATED ? a.N / 2 : tp_cdiv(a.N, 2);
    TP_REQUIRE(tp_cdiv(items, 4) < (1L << 31) && splits <= 65535, "product of few rows: grid too large (N=%d K=%d)", a.N, a.K);
    dim3 grid((unsigned)tp_cdiv(items, 4), splits);
    if (a.M <= 1) gemv_launch_mr<1>(a, grid, part, kps, splits);
    else gemv_launch_mr<2>(a, grid, part, kps, splits);
    return tp_check_launch("linear (few rows)");
}
