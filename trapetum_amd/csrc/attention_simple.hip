// Plain attention kernel for any dtype, head size up to 256 and any grouping: one wave per (row, query head),
// keys visited one after the other in position order with a running softmax.
//
// It is the float32 path's attention for prefill and decode alike (the same instruction sequence per key in
// both, so a token's result does not depend on how the prompt was cut), and the bf16 path's fallback for
// shapes the matrix-core kernels refuse.  Formula and order as the reference's attn_k
// (runtime/cuda/codebook_gemv.cu:240-270): score = dot * scale, cap * tanh(score / cap), softmax, weighted
// sum of v, kv head = head / (heads / kv_heads); the scale is an argument (rsqrt(head_dim) there), and a
// window W hides keys with p - t >= W (none there).
#include "common.h"

struct AttnSimpleArgs {
    const void* q; long q_stride;
    // keys and values of the step itself (prefill): rows of sequence s start at cu_rows[s] and stand at the
    // positions from new_len[s] - count on (from 0 without new_len); row_pos holds every row's position
    const void* k; long k_stride; const void* v; long v_stride;
    const int* cu_rows; const int* row_seq; const int* row_pos;
    // keys and values in the paged cache: all of them in a decode step (sequence i is row i, its last position
    // new_len[i] - 1), the positions before the step's own rows otherwise
    const int* new_len; const int* table; int table_w; const void* k_pool; const void* v_pool; int page; int rows_cap;
    void* out;
    int H, KV, hd; float scale, cap; int window; int paged;
};

template <typename T>
__global__ void __launch_bounds__(64)
attn_simple_k(AttnSimpleArgs a) {
    const int h = blockIdx.y, r = blockIdx.x, lane = threadIdx.x;
    const int g = h / (a.H / a.KV);
    int seq, p, start = 0;                              // start: the first position that is a row of the step
    if (a.paged) { seq = r; p = a.new_len[r] - 1; start = p + 1; }
    else {
        seq = a.row_seq[r];
        p = a.row_pos[r];
        if (a.new_len) start = a.new_len[seq] - (a.cu_rows[seq + 1] - a.cu_rows[seq]);
    }
    const int lo = a.window > 0 ? max(0, p - a.window + 1) : 0;
    const T* q = (const T*)a.q + (size_t)r * a.q_stride + (size_t)h * a.hd;
    float qv[4], o[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int d = lane + 64 * j;
        qv[j] = d < a.hd ? ld_f32(q + d) : 0.f;
        o[j] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    // a key's row and value row are fetched while the two keys before it are worked on (the arithmetic per key, and
    // its order, stay as they are: the loop would otherwise pay a trip to memory, or two through the page table, per key)
    auto fetch = [&](int t, float (&kk)[4], float (&vv)[4]) {
        t = t < p ? t : p;                               // past the last key: a row that exists, never used
        const T *kp, *vp;
        if (t < start) {
            const int row = a.rows_cap > 0 ? t % a.rows_cap : t;
            const int pg = a.table[(size_t)seq * a.table_w + row / a.page];
            const size_t off = (((size_t)pg * a.KV + g) * a.page + row % a.page) * a.hd;
            kp = (const T*)a.k_pool + off;
            vp = (const T*)a.v_pool + off;
        } else {
            const size_t row = (size_t)(a.cu_rows[seq] + t - start);
            kp = (const T*)a.k + row * a.k_stride + (size_t)g * a.hd;
            vp = (const T*)a.v + row * a.v_stride + (size_t)g * a.hd;
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int d = lane + 64 * j;
            const int dc = d < a.hd ? d : 0;
            const float kx = ld_f32(kp + dc), vx = ld_f32(vp + dc);
            kk[j] = d < a.hd ? kx : 0.f;
            vv[j] = d < a.hd ? vx : 0.f;
        }
    };
    auto use = [&](const float (&kk)[4], const float (&vv)[4]) {
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < 4; j++) part = fmaf(qv[j], kk[j], part);
        float s = wave_sum(part) * a.scale;
        if (a.cap > 0.f) s = softcap_f(s, a.cap);
        const float m_new = fmaxf(m, s);
        const float alpha = expf(m - m_new), pr = expf(s - m_new);
        l = l * alpha + pr;
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = o[j] * alpha + pr * vv[j];
        m = m_new;
    };
    float k0[4], v0[4], k1[4], v1[4], k2[4], v2[4];
    fetch(lo, k0, v0);
    fetch(lo + 1, k1, v1);
    for (int t = lo; t <= p; t += 3) {
        fetch(t + 2, k2, v2);
        use(k0, v0);
        if (t + 1 > p) break;
        fetch(t + 3, k0, v0);
        use(k1, v1);
        if (t + 2 > p) break;
        fetch(t + 4, k1, v1);
        use(k2, v2);
    }
    T* out = (T*)a.out + ((size_t)r * a.H + h) * a.hd;
    const float inv = 1.f / l;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int d = lane + 64 * j;
        if (d < a.hd) st_f32(out + d, o[j] * inv);
    }
}

static int launch(const AttnSimpleArgs& a, int dtype, int M, hipStream_t s) {
    TP_REQUIRE(M > 0 && a.H > 0 && a.KV > 0 && a.hd > 0, "attention: empty shape rows=%d heads=%d kv=%d head_dim=%d", M, a.H, a.KV, a.hd);
    TP_REQUIRE(a.H % a.KV == 0, "attention: %d query heads are no multiple of %d kv heads", a.H, a.KV);
    TP_REQUIRE(a.hd <= 256, "attention (plain kernel): head_dim %d exceeds 256", a.hd);
    TP_REQUIRE(a.H <= 65535, "attention (plain kernel): %d heads exceed one launch (65535)", a.H);
    dim3 grid(M, a.H);
    if (dtype == TP_BF16) attn_simple_k<bf16_t><<<grid, 64, 0, s>>>(a);
    else if (dtype == TP_F32) attn_simple_k<float><<<grid, 64, 0, s>>>(a);
    else return tp_fail("attention: unknown dtype %d", dtype);
    return tp_check_launch("attention (plain kernel)");
}

// new_len (or null): the sequences' lengths after the step; the positions before a sequence's first row of the step
// are read from the cache (pools [pages, kv_heads, page, head_dim] through `table`), as earlier steps left it
extern "C" int tp_attn_simple_prefill(const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride,
                                      int dtype, int M, int H, int KV, int hd, const int* cu_rows, const int* row_seq,
                                      const int* row_pos, const int* new_len, const int* table, int table_w,
                                      const void* k_pool, const void* v_pool, int page, int rows_cap,
                                      float scale, float cap, int window, void* out, void* stream) {
    TP_REQUIRE(!new_len || (table && k_pool && v_pool && page > 0 && table_w > 0), "attention: cached positions need the page table and the pools");
    AttnSimpleArgs a{};
    a.q = q; a.q_stride = q_stride; a.k = k; a.k_stride = k_stride; a.v = v; a.v_stride = v_stride;
    a.cu_rows = cu_rows; a.row_seq = row_seq; a.row_pos = row_pos;
    a.new_len = new_len; a.table = table; a.table_w = table_w; a.k_pool = k_pool; a.v_pool = v_pool;
    a.page = new_len ? page : 1; a.rows_cap = new_len ? rows_cap : 0;
    a.out = out; a.H = H; a.KV = KV; a.hd = hd; a.scale = scale; a.cap = cap; a.window = window; a.paged = 0;
    return launch(a, dtype, M, (hipStream_t)stream);
}

extern "C" int tp_attn_simple_decode(const void* q, long q_stride, int dtype, int n_seq, int H, int KV, int hd,
                                     const int* new_len, const int* table, int table_w, const void* k_pool,
                                     const void* v_pool, int page, int rows_cap, float scale, float cap, int window,
                                     void* out, void* stream) {
    TP_REQUIRE(page > 0 && table_w > 0, "attention: page size %d, table width %d", page, table_w);
    AttnSimpleArgs a{};
    a.q = q; a.q_stride = q_stride; a.new_len = new_len; a.table = table; a.table_w = table_w;
    a.k_pool = k_pool; a.v_pool = v_pool; a.page = page; a.rows_cap = rows_cap;
    a.out = out; a.H = H; a.KV = KV; a.hd = hd; a.scale = scale; a.cap = cap; a.window = window; a.paged = 1;
    return launch(a, dtype, n_seq, (hipStream_t)stream);
}
