// bf16 product for three to eight rows (a decode step of a few sequences): bound by reading W once.
//
// What the memory system rewards was measured on MI355X with kernels that only read an [18432, 2304] matrix: blocks
// that ask for their whole region at once, no loop, and whose region is small (8 rows: 5.1 TB/s; 16 rows: 4.8; 32
// rows read in rounds, as the kernel for up to 64 rows does: 3.9), with instructions that take whole 128-byte lines.
// So a block of four waves owns 8 rows of W (a gated product: the 8 gate rows and the 8 up rows of 8 units) and one
// slice of K; wave w takes a quarter of the slice, a step of 64 k an instruction: lane l loads 16 bytes of row l % 8
// at piece l / 8, eight rows by 128 bytes, and the same piece of row l % 8 of X.  Fed to v_mfma_f32_16x16x32_bf16 as
// they are, lane (i = l % 16, g = l / 16) holds piece 2g + i / 8 of row i % 8, of W as A and of X as B, so that
// C[i][j] = sum over g of W[i % 8][piece 2g + i / 8] . X[j % 8][piece 2g + j / 8]: where i / 8 == j / 8 that is the
// half of the dot product over the even or the odd pieces, and C[r][m] + C[r + 8][m + 8] is the whole of it; the other
// half of C is not used.  One instruction per kilobyte of W, as with 16-row tiles, at half the rows and twice the k.
// The four waves' tiles are added in LDS in wave order; K slices go to the workspace as float32 [slices, M, N] for
// the consumer to add in slice order.  No atomics: the order of the sum depends on the shape only (the reference's
// gemv4_partial + gemv_reduce pair has the same property: runtime/cuda/codebook_gemv.cu:86-114, :178-184).
#include "gemm.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

namespace {
constexpr int R8_MAX_STEPS = TP_R8_MAX_STEPS;    // steps of 64 k a wave has in flight at once: a K slice of 2,304 in one go
union Frag8 { uint4 u; bf16x8 v; };
}

// NG: groups of 8 rows of W a block owns (2: gate rows and up rows of the same units); NS: steps of 64 k per wave and round
template <int NG, int NS>
__global__ void __launch_bounds__(256)
gemm_rows8_k(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, void* __restrict__ Y, float* __restrict__ part,
             int M, int N, int K, int k_per_split, int n_splits, int out_dtype, int epilogue, float2 epi, int units) {
    __shared__ float red[4][NG][64][4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 7, piece = lane >> 3;
    const int split = blockIdx.y;
    const int kbeg = split * k_per_split, kend = min(K, kbeg + k_per_split);
    // the block's rows: 8 neighbours, or (gated: the packed matrix alternates 16 gate rows and the 16 up rows of the
    // same units) the gate rows of units 8 b .. 8 b + 7 and their up rows, 16 further on
    int row0[NG];
    if (epilogue == TP_EPI_GATED) {
#pragma unroll
        for (int t = 0; t < NG; t++)
            row0[t] = NG == 4 ? blockIdx.x * 32 + t * 8 : (blockIdx.x >> 1) * 32 + (blockIdx.x & 1) * 8 + t * 16;
    } else {
#pragma unroll
        for (int t = 0; t < NG; t++) row0[t] = (blockIdx.x * NG + t) * 8;
    }
    const bf16_t* wrow[NG];
#pragma unroll
    for (int t = 0; t < NG; t++) wrow[t] = W + (size_t)min(row0[t] + r, N - 1) * K;
    const bool xok = r < M;
    const bf16_t* xrow = X + (size_t)(xok ? r : 0) * K;

    f32x4 acc[NG];
#pragma unroll
    for (int t = 0; t < NG; t++) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // a round: the four waves' quarters of 4 * NS * 64 k, every load of it in flight at once.  Loads are unconditional:
    // past the end of the slice they read its last piece, and X's fragment is zeroed instead.
    const int klast = kend - 8;
    for (int kr = kbeg; kr < kend; kr += 4 * NS * 64) {
        const int k0 = kr + wave * (NS * 64) + piece * 8;
        bf16x8 a[NS][NG], b[NS];
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const int k = k0 + s * 64;
            const bool ok = k < kend;
            const int kc = ok ? k : klast;
#pragma unroll
            for (int t = 0; t < NG; t++) {
                Frag8 f;
                f.u = *reinterpret_cast<const uint4*>(wrow[t] + kc);
                a[s][t] = f.v;
            }
            Frag8 f;
            f.u = *reinterpret_cast<const uint4*>(xrow + kc);
            const uint32_t keep = (uint32_t) - (int)(ok && xok);              // all ones or zero: an AND, not a branch
            f.u.x &= keep; f.u.y &= keep; f.u.z &= keep; f.u.w &= keep;
            b[s] = f.v;
        }
        // every load of the round is asked for before the first product waits for one: the scheduler would otherwise
        // hold loads back to save registers, and the block would no longer read its region in one go
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < NS; s++)
#pragma unroll
            for (int t = 0; t < NG; t++) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s][t], b[s], acc[t], 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < NG; t++)
#pragma unroll
        for (int c = 0; c < 4; c++) red[wave][t][lane][c] = acc[t][c];
    __syncthreads();
    // thread m * 8 + wr: row wr of the block's eight, row m of X.  C[wr][m] lies in lane m + 16 (wr / 4), component
    // wr % 4; C[wr + 8][m + 8] forty lanes further on.  The waves in wave order, in each the even pieces first.
    if (threadIdx.x >= 64) return;
    const int m = threadIdx.x >> 3, wr = threadIdx.x & 7;
    if (m >= M) return;
    const int l0 = m + 16 * (wr >> 2), c = wr & 3;
    float v[NG];
#pragma unroll
    for (int t = 0; t < NG; t++) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) s += red[w][t][l0][c] + red[w][t][l0 + 40][c];
        v[t] = s;
    }
    if (n_splits > 1) {
#pragma unroll
        for (int t = 0; t < NG; t++)
            if (row0[t] + wr < N) part[((size_t)split * M + m) * N + row0[t] + wr] = v[t];
    } else if (NG >= 2 && epilogue == TP_EPI_GATED) {
#pragma unroll
        for (int p = 0; p < NG / 2; p++) {
            const int unit = blockIdx.x * (NG * 4) + p * 8 + wr;
            if (unit >= units) continue;
            const float o = gate_act_fast(v[p], epi) * v[p + NG / 2];
            if (out_dtype == TP_F32) ((float*)Y)[(size_t)m * units + unit] = o;
            else ((bf16_t*)Y)[(size_t)m * units + unit] = f32_to_bf16(o);
        }
    } else {
#pragma unroll
        for (int t = 0; t < NG; t++) {
            const int n = row0[t] + wr;
            if (n >= N) continue;
            float o = v[t];
            if (epilogue == TP_EPI_SOFTCAP) o = softcap_f(o, epi.x);
            if (out_dtype == TP_F32) ((float*)Y)[(size_t)m * N + n] = o;
            else ((bf16_t*)Y)[(size_t)m * N + n] = f32_to_bf16(o);
        }
    }
}

bool gemm_rows8_supports(const GemmArgs& a) {
    return a.in_dtype == TP_BF16 && a.M <= 8 && a.K % 8 == 0 && (a.epilogue != TP_EPI_GATED || a.N % 32 == 0);
}

// Groups of 8 rows a block owns.  Every group shares the block's fragments of X, whose loads compete with W's (measured
// at the 2B shapes, 8 rows of X: without them the products run 0.5 to 5 us shorter), but a larger region per block reads
// slower and leaves fewer blocks: as many groups as still leave about three blocks a CU, K slices counted.
static int rows8_groups(const GemmArgs& a) {
    if (a.epilogue == TP_EPI_GATED) return 2;
    const int most = a.defer && a.epilogue == TP_EPI_NONE && a.K / 512 > 1 ? a.K / 512 : 1;
    if (!a.defer) return (long)tp_cdiv(a.N, 16) >= 256 ? 2 : 1;
    for (int g = 4; g > 1; g >>= 1)             // (2B step of 8 sequences with at most 4 / 2 / 1 groups: 2.001 / 2.024 / 2.062 ms)
        if ((long)tp_cdiv(a.N, 8 * g) * most >= 3 * 256) return g;      // three blocks for each of the chip's 256 CUs
    return 1;
}

// K slices where the consumer adds them: enough for about four blocks a CU, none shorter than 512
static void rows8_plan(const GemmArgs& a, int& blocks, int& splits, int& kps) {
    blocks = tp_cdiv(a.N, 8 * rows8_groups(a));
    splits = 1;
    if (a.epilogue == TP_EPI_NONE && a.defer) {
        const int want = tp_cdiv(1024, blocks), most = a.K / 512 > 1 ? a.K / 512 : 1;
        splits = want < most ? want : most;
    }
    kps = tp_cdiv(tp_cdiv(a.K, splits), 256) * 256;
    splits = tp_cdiv(a.K, kps);
}

size_t gemm_rows8_workspace(const GemmArgs& a) {
    int blocks, splits, kps;
    rows8_plan(a, blocks, splits, kps);
    return splits > 1 ? (size_t)splits * a.M * a.N * sizeof(float) : 0;
}

template <int NG, int NS>
static void rows8_launch_ns(const GemmArgs& a, dim3 grid, float* part, int kps, int splits) {
    gemm_rows8_k<NG, NS><<<grid, 256, 0, a.stream>>>((const bf16_t*)a.x, (const bf16_t*)a.w, a.y, part, a.M, a.N, a.K, kps, splits,
                                                     a.out_dtype, a.epilogue, epi_constants(a), a.units);
}

template <int NG>
static void rows8_launch_ng(const GemmArgs& a, int ns, dim3 grid, float* part, int kps, int splits) {
    switch (ns) {
        case 1: rows8_launch_ns<NG, 1>(a, grid, part, kps, splits); break;
        case 2: rows8_launch_ns<NG, 2>(a, grid, part, kps, splits); break;
        case 3: rows8_launch_ns<NG, 3>(a, grid, part, kps, splits); break;
        case 4: rows8_launch_ns<NG, 4>(a, grid, part, kps, splits); break;
        case 5: rows8_launch_ns<NG, 5>(a, grid, part, kps, splits); break;
        case 6: rows8_launch_ns<NG, 6>(a, grid, part, kps, splits); break;
        case 7: rows8_launch_ns<NG, 7>(a, grid, part, kps, splits); break;
        case 8: rows8_launch_ns<NG, 8>(a, grid, part, kps, splits); break;
        default: rows8_launch_ns<NG, R8_MAX_STEPS>(a, grid, part, kps, splits); break;
    }
}

int gemm_rows8_launch(const GemmArgs& a) {
    TP_REQUIRE(gemm_rows8_supports(a), "product of a few rows: needs bf16, at most 8 rows and K a multiple of 8 (M=%d N=%d K=%d)", a.M, a.N, a.K);
    TP_REQUIRE(((uintptr_t)a.x % 16 == 0) && ((uintptr_t)a.w % 16 == 0), "product of a few rows: operands must be 16-byte aligned");
    int blocks, splits, kps;
    rows8_plan(a, blocks, splits, kps);
    float* part = nullptr;
    if (splits > 1) {
        const size_t need = (size_t)splits * a.M * a.N * sizeof(float);
        TP_REQUIRE(a.workspace && a.workspace_bytes >= need, "product of a few rows: workspace of %zu bytes, %zu needed", a.workspace_bytes, need);
        part = (float*)a.workspace;
    }
    TP_REQUIRE(splits <= 65535, "product of a few rows: too many K slices (K=%d)", a.K);
    // steps per wave and round: the slice in as few rounds as the registers allow, the rounds of equal length
    const int steps = tp_cdiv(kps, 256);
    const int rounds = tp_cdiv(steps, R8_MAX_STEPS);
    const int ns = tp_cdiv(steps, rounds);
    dim3 grid(blocks, splits);
    if (rows8_groups(a) == 4) rows8_launch_ng<4>(a, ns, grid, part, kps, splits);
    else if (rows8_groups(a) == 2) rows8_launch_ng<2>(a, ns, grid, part, kps, splits);
    else rows8_launch_ng<1>(a, ns, grid, part, kps, splits);
    return tp_check_launch("linear (a few rows)");
}
