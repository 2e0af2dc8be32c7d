// bf16 product for at most 64 rows (decode steps, logits of a few rows): bound by reading W once.
//
// A block of four waves owns 16 (or 32) rows of W and one slice of K; wave w takes the 32-wide k chunks
// w, w+4, ... of the slice, so the four waves together read 256 contiguous bytes of every W row per
// round.  W rows are the A operand of v_mfma_f32_16x16x32_bf16 (lane l holds 8 consecutive k of row
// l % 16), the step's rows X the B operand, so each lane loads 16 bytes straight from global memory
// into its operand registers: no LDS staging, nothing but W streams from HBM.  The waves' partial
// tiles are added in LDS in wave order; K slices (when N alone cannot fill 256 CUs) go to a workspace
// and are added in slice order by a second kernel.  No atomics: the sum's order depends on the shape
// only (the reference's gemv4_partial + gemv_reduce pair has the same property:
// runtime/cuda/codebook_gemv.cu:86-114, :178-184).
#include "gemm.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

union Frag { uint4 u; bf16x8 v; };

__device__ __forceinline__ bf16x8 load_frag(const bf16_t* p, bool ok) {
    Frag f;
    if (ok) f.u = *reinterpret_cast<const uint4*>(p);
    else f.u = make_uint4(0, 0, 0, 0);
    return f.v;
}

__device__ __forceinline__ void store_out(void* y, int out_dtype, size_t idx, float v) {
    if (out_dtype == TP_F32) ((float*)y)[idx] = v;
    else ((bf16_t*)y)[idx] = f32_to_bf16(v);
}

// MT: 16-row tiles of X (rows padded to 16 * MT); NT: 16-row tiles of W per block, all fed by the same X
// fragments (a gated product needs an even number: gate tile and up tile of the same 16 units alternate).
template <int MT, int NT>
__global__ void __launch_bounds__(256)
gemm_skinny_k(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, void* __restrict__ Y, float* __restrict__ part,
              int M, int N, int K, int k_per_split, int n_splits, int out_dtype, int epilogue, float2 epi, int units) {
    __shared__ float red[4][MT][64][4];                   // one W tile's partial tiles of the four waves at a time
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * (16 * NT);
    const int split = blockIdx.y;
    const int kbeg = split * k_per_split;
    const int kend = min(K, kbeg + k_per_split);

    const bf16_t* wrow[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        int n = n0 + t * 16 + r;
        if (n >= N) n = N - 1;
        wrow[t] = W + (size_t)n * K;
    }
    const bf16_t* xrow[MT];
    bool xok[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) {
        const int m = t * 16 + r;
        xok[t] = m < M;
        xrow[t] = X + (size_t)(xok[t] ? m : 0) * K;
    }

    f32x4 acc[NT][MT];
#pragma unroll
    for (int a = 0; a < NT; a++)
#pragma unroll
        for (int b = 0; b < MT; b++) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // Two register sets of U rounds each: while one set feeds the products, the loads of the next U rounds are
    // in flight.  Loads are unconditional (a branch around a load would make the compiler wait for it at the
    // join): past the end of the slice they read the slice's last chunk and X's fragment is zeroed instead.
    constexpr int U = MT >= 4 ? 2 : 4;
    union FragU { uint4 u; bf16x8 v; };
    const int klast = kend - 8;
    auto load = [&](int kw, bf16x8 (&a)[U][NT], bf16x8 (&b)[U][MT]) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = kw + (u >> 1) * 256 + (u & 1) * 32 + g * 8;
            const bool ok = k < kend;
            const int kc = ok ? k : klast;
#pragma unroll
            for (int t = 0; t < NT; t++) {
                FragU f;
                f.u = *reinterpret_cast<const uint4*>(wrow[t] + kc);
                a[u][t] = f.v;
            }
#pragma unroll
            for (int t = 0; t < MT; t++) {
                FragU f;
                f.u = *reinterpret_cast<const uint4*>(xrow[t] + kc);
                const uint32_t keep = (uint32_t) - (int)(ok && xok[t]);      // all ones or zero: an AND, not a branch
                f.u.x &= keep; f.u.y &= keep; f.u.z &= keep; f.u.w &= keep;
                b[u][t] = f.v;
            }
        }
    };
    auto mma = [&](bf16x8 (&a)[U][NT], bf16x8 (&b)[U][MT]) {
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int s = 0; s < NT; s++)
#pragma unroll
                for (int t = 0; t < MT; t++)
                    acc[s][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][s], b[u][t], acc[s][t], 0, 0, 0);
    };
    bf16x8 a0[U][NT], b0[U][MT], a1[U][NT], b1[U][MT];
    int kw = kbeg + wave * 64;
    if (kw < kend) {
        load(kw, a0, b0);
        while (true) {
            load(kw + 128 * U, a1, b1);
            mma(a0, b0);
            kw += 128 * U;
            if (kw >= kend) break;
            load(kw + 128 * U, a0, b0);
            mma(a1, b1);
            kw += 128 * U;
            if (kw >= kend) break;
        }
    }

    // thread -> one element of every tile: lane l2 = tid / 4, component i = tid % 4
    const int l2 = threadIdx.x >> 2, i = threadIdx.x & 3;
    const int nl = (l2 >> 4) * 4 + i;                     // W row within the tile
    const int ml = l2 & 15;                               // X row within the tile
    float v[MT][NT];
#pragma unroll
    for (int s = 0; s < NT; s++) {                        // the waves' partial tiles are added in wave order
        if (s > 0) __syncthreads();
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int c = 0; c < 4; c++) red[wave][t][lane][c] = acc[s][t][c];
        __syncthreads();
#pragma unroll
        for (int t = 0; t < MT; t++)
            v[t][s] = ((red[0][t][l2][i] + red[1][t][l2][i]) + red[2][t][l2][i]) + red[3][t][l2][i];
    }

#pragma unroll
    for (int t = 0; t < MT; t++) {
        const int m = t * 16 + ml;
        if (m >= M) continue;
        if (n_splits > 1) {
#pragma unroll
            for (int s = 0; s < NT; s++) {
                const int n = n0 + s * 16 + nl;
                if (n < N) part[((size_t)split * M + m) * N + n] = v[t][s];
            }
        } else if (NT >= 2 && epilogue == TP_EPI_GATED) {
#pragma unroll
            for (int s = 0; s + 1 < NT; s += 2) {         // tiles alternate: 16 gate rows, the 16 up rows of the same units
                const int unit = ((n0 + s * 16) >> 1) + nl;
                if (unit < units) store_out(Y, out_dtype, (size_t)m * units + unit, gate_act_fast(v[t][s], epi) * v[t][s + 1]);
            }
        } else {
#pragma unroll
            for (int s = 0; s < NT; s++) {
                const int n = n0 + s * 16 + nl;
                if (n >= N) continue;
                float o = v[t][s];
                if (epilogue == TP_EPI_SOFTCAP) o = softcap_f(o, epi.x);
                store_out(Y, out_dtype, (size_t)m * N + n, o);
            }
        }
    }
}

// adds the K slices in slice order and applies the epilogue
__global__ void skinny_reduce_k(const float* __restrict__ part, void* __restrict__ Y, int M, int N, int n_splits,
                                int out_dtype, int epilogue, float2 epi, int units) {
    const int cols = epilogue == TP_EPI_GATED ? units : N;
    const long total = (long)M * cols;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int m = (int)(idx / cols), c = (int)(idx % cols);
        if (epilogue == TP_EPI_GATED) {
            const int ng = (c >> 4) * 32 + (c & 15);
            float gsum = 0.f, usum = 0.f;
            for (int s = 0; s < n_splits; s++) {
                const float* p = part + ((size_t)s * M + m) * N;
                gsum += p[ng];
                usum += p[ng + 16];
            }
            store_out(Y, out_dtype, idx, gate_act_fast(gsum, epi) * usum);
        } else {
            float sum = 0.f;
            for (int s = 0; s < n_splits; s++) sum += part[((size_t)s * M + m) * N + c];
            if (epilogue == TP_EPI_SOFTCAP) sum = softcap_f(sum, epi.x);
            store_out(Y, out_dtype, idx, sum);
        }
    }
}

bool gemm_skinny_supports(const GemmArgs& a) {
    return a.in_dtype == TP_BF16 && a.M <= 64 && a.K % 8 == 0;
}

static void plan(const GemmArgs& a, int& nt, int& blocks, int& splits, int& k_per_split) {
    // W tiles per block: every tile reuses the block's X fragments, so more tiles mean less X traffic per byte
    // of W (which matters from 16 rows on), as long as tiles x K slices still fill the chip
    const int gated = a.epilogue == TP_EPI_GATED;
    const int kslices = a.K / 512 > 1 ? a.K / 512 : 1;
    nt = gated ? 2 : 1;
    if (a.M > 16) {
        if ((long)tp_cdiv(a.N, 64) * kslices >= 512) nt = 4;
        else if ((long)tp_cdiv(a.N, 32) * kslices >= 512) nt = 2;
    } else if (a.N >= 65536) {
        nt = 2;
    }
    blocks = tp_cdiv(a.N, 16 * nt);
    int want = tp_cdiv(512, blocks);
    int most = a.K / 512;
    if (most < 1) most = 1;
    splits = want < most ? want : most;
    if (splits < 1) splits = 1;
    k_per_split = tp_cdiv(tp_cdiv(a.K, splits), 128) * 128;
    splits = tp_cdiv(a.K, k_per_split);
}

size_t gemm_skinny_workspace(const GemmArgs& a) {
    int nt, blocks, splits, kps;
    plan(a, nt, blocks, splits, kps);
    return splits > 1 ? (size_t)splits * a.M * a.N * sizeof(float) : 0;
}

template <int MT>
static void launch_mt(const GemmArgs& a, int nt, dim3 grid, float* part, int kps, int splits) {
    if (nt == 4)
        gemm_skinny_k<MT, 4><<<grid, 256, 0, a.stream>>>((const bf16_t*)a.x, (const bf16_t*)a.w, a.y, part, a.M, a.N, a.K,
                                                         kps, splits, a.out_dtype, a.epilogue, epi_constants(a), a.units);
    else if (nt == 2)
        gemm_skinny_k<MT, 2><<<grid, 256, 0, a.stream>>>((const bf16_t*)a.x, (const bf16_t*)a.w, a.y, part, a.M, a.N, a.K,
                                                         kps, splits, a.out_dtype, a.epilogue, epi_constants(a), a.units);
    else
        gemm_skinny_k<MT, 1><<<grid, 256, 0, a.stream>>>((const bf16_t*)a.x, (const bf16_t*)a.w, a.y, part, a.M, a.N, a.K,
                                                         kps, splits, a.out_dtype, a.epilogue, epi_constants(a), a.units);
}

int gemm_skinny_launch(const GemmArgs& a) {
    TP_REQUIRE(gemm_skinny_supports(a), "skinny product: needs bf16, at most 64 rows and K a multiple of 8 (M=%d K=%d)", a.M, a.K);
    TP_REQUIRE(((uintptr_t)a.x % 16 == 0) && ((uintptr_t)a.w % 16 == 0), "skinny product: operands must be 16-byte aligned");
    int nt, blocks, splits, kps;
    plan(a, nt, blocks, splits, kps);
    float* part = nullptr;
    if (splits > 1) {
        const size_t need = (size_t)splits * a.M * a.N * sizeof(float);
        TP_REQUIRE(a.workspace && a.workspace_bytes >= need, "skinny product: workspace of %zu bytes, %zu needed", a.workspace_bytes, need);
        part = (float*)a.workspace;
    }
    dim3 grid(blocks, splits);
    if (a.M <= 16) launch_mt<1>(a, nt, grid, part, kps, splits);
    else if (a.M <= 32) launch_mt<2>(a, nt, grid, part, kps, splits);
    else launch_mt<4>(a, nt, grid, part, kps, splits);
    if (int rc = tp_check_launch("linear (skinny kernel)")) return rc;
    if (splits > 1 && !a.defer) {
        const long total = (long)a.M * (a.epilogue == TP_EPI_GATED ? a.units : a.N);
        int rb = tp_cdiv(total, 256);
        if (rb > 2048) rb = 2048;
        skinny_reduce_k<<<rb, 256, 0, a.stream>>>(part, a.y, a.M, a.N, splits, a.out_dtype, a.epilogue, epi_constants(a), a.units);
        return tp_check_launch("linear (skinny reduce)");
    }
    return 0;
}
