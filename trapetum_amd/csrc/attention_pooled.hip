// Attention over a window of tokens plus one pooled key and value per block of tokens that lies wholly before the
// window, with the heads' softmax weights mixed by a matrix ("talking heads"); and what feeds it.
//
//   qkv_prepare     one launch for a step's projected rows: bias, rotation of a head's leading elements, division of
//                   every query and key head by its root mean square (a norm without a gain), rounding to the
//                   activation dtype; everything in float32 from the product's sums
//   pool_write      the mean key and mean value of every block of P positions that the step completes, into a paged
//                   pool that keeps one row per block; the sums of a block that the step leaves unfinished wait in a
//                   float32 state of the sequence, so the additions run in position order however a prompt is cut
//   attn_pooled     the query at position p sees the blocks b with (b + 1) P <= p - W + 1 and the positions
//                   max(0, p - W + 1) .. p; one softmax over both; score = cap tanh(q . k scale / cap)
//   talk_mix        out_h = sum_g T[h, g] A[g, kv(h)], A[g, c] being head g's weights applied to the values of kv head c
//
// The mixed weights of head h meet the values of h's own kv head, so head h needs, of every head g, g's weights
// applied to the values of kv(h): the attention is computed for every pair (g, c) of a query head and a kv head whose
// values it weighs, and the mix is a small product over g afterwards.  The plain kernel gives a wave one such pair of
// one row and visits the keys one after the other in position order (pooled blocks first) with a running softmax:
// the same instruction sequence per key whether a position is decoded alone or stands in a prompt.
#include "common.h"

// ---- bias, rotation, unit norm ---------------------------------------------------------------------------------------
// grid (rows, heads): a wave per head of the row (query heads, then key heads, then value heads).  Elements of a
// head beyond `dim` (or `vdim`) are the zero filling of rows that keep keys and values at one size.
template <typename TI, typename TO>
__global__ void __launch_bounds__(64)
qkv_prepare_k(const TI* __restrict__ x, long x_stride, const float* __restrict__ bias, int H, int KV, int row, int dim,
              const float* __restrict__ inv_freq, int rot, int pairing, float unit_eps, const int* __restrict__ row_pos,
              TO* __restrict__ q, TO* __restrict__ k, TO* __restrict__ v) {
    const int r = blockIdx.x, j = blockIdx.y, lane = threadIdx.x;
    const TI* src = x + (size_t)r * x_stride + (size_t)j * row;
    const float* b = bias ? bias + (size_t)j * row : nullptr;
    TO* dst = j < H ? q + ((size_t)r * H + j) * row : (j < H + KV ? k + ((size_t)r * KV + (j - H)) * row : v + ((size_t)r * KV + (j - H - KV)) * row);
    if (j >= H + KV) {                                   // a value head: the bias, nothing else
        for (int d = lane; d < row; d += 64) st_f32(dst + d, ld_f32(src + d) + (b ? b[d] : 0.f));
        return;
    }
    const float pos = (float)row_pos[r];
    const int half = rot / 2;
    float ss = 0.f;
    // pairs that turn together, then the elements that pass; the sum of squares does not change under the rotation,
    // it is taken of the turned values as they are stored
    for (int f = lane; f < half; f += 64) {
        const int e0 = pairing == TP_ROPE_NEIGHBOURS ? 2 * f : f, e1 = pairing == TP_ROPE_NEIGHBOURS ? 2 * f + 1 : f + half;
        const float ang = pos * inv_freq[f];
        const float c = cosf(ang), sn = sinf(ang);
        const float x0 = ld_f32(src + e0) + (b ? b[e0] : 0.f), x1 = ld_f32(src + e1) + (b ? b[e1] : 0.f);
        const float y0 = x0 * c - x1 * sn, y1 = x1 * c + x0 * sn;
        ss += y0 * y0 + y1 * y1;
    }
    for (int d = rot + lane; d < dim; d += 64) { const float y = ld_f32(src + d) + (b ? b[d] : 0.f); ss = __builtin_fmaf(y, y, ss); }
    const float inv = unit_eps >= 0.f ? rsqrtf(wave_sum(ss) / (float)dim + unit_eps) : 1.f;
    for (int f = lane; f < half; f += 64) {
        const int e0 = pairing == TP_ROPE_NEIGHBOURS ? 2 * f : f, e1 = pairing == TP_ROPE_NEIGHBOURS ? 2 * f + 1 : f + half;
        const float ang = pos * inv_freq[f];
        const float c = cosf(ang), sn = sinf(ang);
        const float x0 = ld_f32(src + e0) + (b ? b[e0] : 0.f), x1 = ld_f32(src + e1) + (b ? b[e1] : 0.f);
        st_f32(dst + e0, (x0 * c - x1 * sn) * inv);
        st_f32(dst + e1, (x1 * c + x0 * sn) * inv);
    }
    for (int d = rot + lane; d < row; d += 64) st_f32(dst + d, d < dim ? (ld_f32(src + d) + (b ? b[d] : 0.f)) * inv : 0.f);
}

extern "C" int tp_qkv_prepare(const void* x, long x_stride, int in_dtype, const float* bias, int M, int H, int KV, int row, int dim,
                              const float* inv_freq, int rot, int pairing, float unit_eps, const int* row_pos,
                              void* q, void* k, void* v, int out_dtype, void* stream) {
    TP_REQUIRE(M > 0 && H > 0 && KV >= 0 && row > 0 && dim > 0 && dim <= row, "qkv_prepare: empty shape rows=%d heads=%d kv=%d row=%d dim=%d", M, H, KV, row, dim);
    TP_REQUIRE(rot >= 0 && rot <= dim && rot % 2 == 0, "qkv_prepare: a rotation over %d elements must be even and at most %d", rot, dim);
    TP_REQUIRE(rot == 0 || inv_freq, "qkv_prepare: a rotation needs its frequency table");
    TP_REQUIRE(pairing == TP_ROPE_HALVES || pairing == TP_ROPE_NEIGHBOURS, "qkv_prepare: unknown pairing %d", pairing);
    TP_REQUIRE(x && q && row_pos && (KV == 0 || (k && v)), "qkv_prepare: null operand");
    TP_REQUIRE(x_stride >= (long)(H + 2 * KV) * row, "qkv_prepare: rows of %ld elements are too short for %d heads of %d", x_stride, H + 2 * KV, row);
    TP_REQUIRE(H + 2 * KV <= 65535, "qkv_prepare: %d heads exceed one launch", H + 2 * KV);
    dim3 grid(M, H + 2 * KV);
    hipStream_t s = (hipStream_t)stream;
#define TP_QKV(TI, TO) qkv_prepare_k<TI, TO><<<grid, 64, 0, s>>>((const TI*)x, x_stride, bias, H, KV, row, dim, inv_freq, rot, pairing, unit_eps, row_pos, (TO*)q, (TO*)k, (TO*)v)
    if (in_dtype == TP_F32 && out_dtype == TP_F32) TP_QKV(float, float);
    else if (in_dtype == TP_F32 && out_dtype == TP_BF16) TP_QKV(float, bf16_t);
    else if (in_dtype == TP_BF16 && out_dtype == TP_BF16) TP_QKV(bf16_t, bf16_t);
    else return tp_fail("qkv_prepare: no kernel from dtype %d to dtype %d", in_dtype, out_dtype);
#undef TP_QKV
    return tp_check_launch("qkv_prepare");
}

// ---- means of completed blocks ---------------------------------------------------------------------------------------
// grid (sequences, blocks a sequence's rows can touch, pieces of 256 channels); channels: the row's keys, then its values.
// Block index 0 of a sequence takes the block that the step's first row falls into (it may go on from the state) and
// also the block of the step's last row (it may stay unfinished and go into the state), so one thread reads and
// writes a channel of the state; the other indices take the whole blocks in between.
template <typename T>
__global__ void __launch_bounds__(256)
pool_write_k(const T* __restrict__ k, long k_stride, const T* __restrict__ v, long v_stride, int C, int KV, int row, int P,
             const int* __restrict__ cu_rows, const int* __restrict__ new_len, const int* __restrict__ slot_ids,
             float* __restrict__ state, const int* __restrict__ table, int table_w, T* __restrict__ pk, T* __restrict__ pv, int page) {
    const int seq = blockIdx.x, c = blockIdx.z * 256 + threadIdx.x;
    if (c >= 2 * C) return;
    const int first_row = cu_rows[seq], count = cu_rows[seq + 1] - first_row, end = new_len[seq], start = end - count;
    const int b_first = start / P, b_last = (end - 1) / P;
    float* st = state + (size_t)slot_ids[seq] * 2 * C + c;
    const bool is_v = c >= C;
    const int cc = is_v ? c - C : c;
    const T* src = is_v ? v : k;
    const long stride = is_v ? v_stride : k_stride;
    auto one = [&](int b) {
        const int f = b * P, lo = max(f, start), hi = min(f + P, end);
        float acc = f < start ? *st : 0.f;
        for (int t = lo; t < hi; t++) acc += ld_f32(src + (size_t)(first_row + t - start) * stride + cc);
        if (hi == f + P) {
            const int pg = table[(size_t)seq * table_w + b / page];
            if (pg >= 0) {
                T* dst = (is_v ? pv : pk) + (((size_t)pg * KV + cc / row) * page + b % page) * row + cc % row;
                st_f32(dst, acc / (float)P);
            }
        } else *st = acc;
    };
    if (blockIdx.y == 0) {
        one(b_first);
        if (b_last != b_first) one(b_last);
    } else {
        const int b = b_first + blockIdx.y;
        if (b < b_last) one(b);
    }
}

extern "C" int tp_pool_write(const void* k, long k_stride, const void* v, long v_stride, int dtype, int n_seq, int max_count, int KV, int row, int P,
                             const int* cu_rows, const int* new_len, const int* slot_ids, float* state, const int* table, int table_w,
                             void* pk, void* pv, int page, void* stream) {
    TP_REQUIRE(n_seq > 0 && max_count > 0 && KV > 0 && row > 0 && P > 0 && page > 0 && table_w > 0, "pool_write: empty shape");
    TP_REQUIRE(k && v && cu_rows && new_len && slot_ids && state && table && pk && pv, "pool_write: null operand");
    const int C = KV * row;
    TP_REQUIRE(k_stride >= C && v_stride >= C, "pool_write: rows are too short for %d heads of %d", KV, row);
    const int blocks = (max_count + P - 1) / P + 1;       // a run of `count` positions touches at most that many blocks
    TP_REQUIRE(blocks <= 65535, "pool_write: %d blocks of %d positions exceed one launch", blocks, P);
    dim3 grid(n_seq, blocks, tp_cdiv(2 * C, 256));
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TP_BF16) pool_write_k<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)k, k_stride, (const bf16_t*)v, v_stride, C, KV, row, P, cu_rows, new_len, slot_ids, state, table, table_w, (bf16_t*)pk, (bf16_t*)pv, page);
    else if (dtype == TP_F32) pool_write_k<float><<<grid, 256, 0, s>>>((const float*)k, k_stride, (const float*)v, v_stride, C, KV, row, P, cu_rows, new_len, slot_ids, state, table, table_w, (float*)pk, (float*)pv, page);
    else return tp_fail("pool_write: unknown dtype %d", dtype);
    return tp_check_launch("pool_write");
}

// ---- the plain attention kernel ---------------------------------------------------------------------------------------
struct AttnPooledArgs {
    const void* q; long q_stride;
    const void* k; long k_stride; const void* v; long v_stride;       // the step's own rows
    const int* cu_rows; const int* row_seq; const int* row_pos; const int* new_len;
    const int* table; int table_w; const void* k_pool; const void* v_pool; int page; int rows_cap;       // positions before the step
    const int* ptable; int ptable_w; const void* pk; const void* pv; int P;                              // pooled blocks (P 0: none)
    float* out;                                                       // [rows, H, VG, hd] float32
    int H, KV, hd, VG; float scale, cap; int window;
};

template <typename T, int NJ>
__global__ void __launch_bounds__(64)
attn_pooled_k(AttnPooledArgs a) {
    const int r = blockIdx.x, h = blockIdx.y, c = blockIdx.z, lane = threadIdx.x;
    const int gk = h / (a.H / a.KV), gv = a.VG > 1 ? c : gk;
    const int seq = a.row_seq[r], p = a.row_pos[r];
    const int start = a.new_len[seq] - (a.cu_rows[seq + 1] - a.cu_rows[seq]);     // the first position that is a row of the step
    const int lo = a.window > 0 ? max(0, p - a.window + 1) : 0;
    const int nb = (a.P > 0 && a.window > 0) ? max(0, p - a.window + 1) / a.P : 0;
    const int n = nb + p - lo + 1;                      // keys in all: blocks, then positions
    const T* q = (const T*)a.q + (size_t)r * a.q_stride + (size_t)h * a.hd;
    float qv[NJ], o[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int d = lane + 64 * j;
        qv[j] = d < a.hd ? ld_f32(q + d) : 0.f;
        o[j] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    auto fetch = [&](int u, float (&kk)[NJ], float (&vv)[NJ]) {
        u = u < n ? u : n - 1;                           // past the last key: a row that exists, never used
        const T *kp, *vp;
        if (u < nb) {
            const int pg = a.ptable[(size_t)seq * a.ptable_w + u / a.page];
            const size_t at = (size_t)pg * a.KV * a.page + u % a.page;
            kp = (const T*)a.pk + (at + (size_t)gk * a.page) * a.hd;
            vp = (const T*)a.pv + (at + (size_t)gv * a.page) * a.hd;
        } else {
            const int t = lo + u - nb;
            if (t < start) {
                const int row = a.rows_cap > 0 ? t % a.rows_cap : t;
                const int pg = a.table[(size_t)seq * a.table_w + row / a.page];
                const size_t at = (size_t)pg * a.KV * a.page + row % a.page;
                kp = (const T*)a.k_pool + (at + (size_t)gk * a.page) * a.hd;
                vp = (const T*)a.v_pool + (at + (size_t)gv * a.page) * a.hd;
            } else {
                const size_t row = (size_t)(a.cu_rows[seq] + t - start);
                kp = (const T*)a.k + row * a.k_stride + (size_t)gk * a.hd;
                vp = (const T*)a.v + row * a.v_stride + (size_t)gv * a.hd;
            }
        }
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int d = lane + 64 * j;
            const int dc = d < a.hd ? d : 0;
            const float kx = ld_f32(kp + dc), vx = ld_f32(vp + dc);
            kk[j] = d < a.hd ? kx : 0.f;
            vv[j] = d < a.hd ? vx : 0.f;
        }
    };
    auto use = [&](const float (&kk)[NJ], const float (&vv)[NJ]) {
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; j++) part = fmaf(qv[j], kk[j], part);
        float s = wave_sum(part) * a.scale;
        if (a.cap > 0.f) s = softcap_f(s, a.cap);
        const float m_new = fmaxf(m, s);
        const float alpha = expf(m - m_new), pr = expf(s - m_new);
        l = l * alpha + pr;
#pragma unroll
        for (int j = 0; j < NJ; j++) o[j] = o[j] * alpha + pr * vv[j];
        m = m_new;
    };
    float k0[NJ], v0[NJ], k1[NJ], v1[NJ], k2[NJ], v2[NJ];
    fetch(0, k0, v0);
    fetch(1, k1, v1);
    for (int u = 0; u < n; u += 3) {
        fetch(u + 2, k2, v2);
        use(k0, v0);
        if (u + 1 >= n) break;
        fetch(u + 3, k0, v0);
        use(k1, v1);
        if (u + 2 >= n) break;
        fetch(u + 4, k1, v1);
        use(k2, v2);
    }
    float* out = a.out + (((size_t)r * a.H + h) * a.VG + c) * a.hd;
    const float inv = 1.f / l;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int d = lane + 64 * j;
        if (d < a.hd) out[d] = o[j] * inv;
    }
}

// all_values: every query head's weights are applied to the values of every kv head (out [rows, H, KV, hd]), else to
// its own kv head's only (out [rows, H, 1, hd]).  P 0: no pooled blocks.
extern "C" int tp_attn_pooled(const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride, int dtype,
                              int M, int H, int KV, int hd, const int* cu_rows, const int* row_seq, const int* row_pos, const int* new_len,
                              const int* table, int table_w, const void* k_pool, const void* v_pool, int page, int rows_cap,
                              const int* ptable, int ptable_w, const void* pk, const void* pv, int P,
                              float scale, float cap, int window, int all_values, float* out, void* stream) {
    TP_REQUIRE(M > 0 && H > 0 && KV > 0 && hd > 0, "attention (pooled): empty shape rows=%d heads=%d kv=%d head_dim=%d", M, H, KV, hd);
    TP_REQUIRE(H % KV == 0, "attention (pooled): %d query heads are no multiple of %d kv heads", H, KV);
    TP_REQUIRE(hd <= 1024, "attention (pooled, plain kernel): head_dim %d exceeds 1024", hd);
    TP_REQUIRE(H <= 65535 && KV <= 65535, "attention (pooled): %d heads exceed one launch", H);
    TP_REQUIRE(q && k && v && cu_rows && row_seq && row_pos && new_len && out, "attention (pooled): null operand");
    TP_REQUIRE(table && k_pool && v_pool && page > 0 && table_w > 0, "attention (pooled): cached positions need the page table and the pools");
    TP_REQUIRE(rows_cap >= 0 && (rows_cap == 0 || rows_cap % page == 0), "attention (pooled): ring of %d rows is no multiple of the page size %d", rows_cap, page);
    TP_REQUIRE(P >= 0 && (P == 0 || (window > 0 && ptable && pk && pv && ptable_w > 0)), "attention (pooled): blocks of %d positions need a window, their page table and pools", P);
    AttnPooledArgs a{};
    a.q = q; a.q_stride = q_stride; a.k = k; a.k_stride = k_stride; a.v = v; a.v_stride = v_stride;
    a.cu_rows = cu_rows; a.row_seq = row_seq; a.row_pos = row_pos; a.new_len = new_len;
    a.table = table; a.table_w = table_w; a.k_pool = k_pool; a.v_pool = v_pool; a.page = page; a.rows_cap = rows_cap;
    a.ptable = ptable; a.ptable_w = ptable_w; a.pk = pk; a.pv = pv; a.P = P;
    a.out = out; a.H = H; a.KV = KV; a.hd = hd; a.VG = all_values ? KV : 1; a.scale = scale; a.cap = cap; a.window = window;
    dim3 grid(M, H, a.VG);
    hipStream_t s = (hipStream_t)stream;
    if (dtype != TP_BF16 && dtype != TP_F32) return tp_fail("attention (pooled): unknown dtype %d", dtype);
#define TP_ATTN_POOLED(NJ) do { if (dtype == TP_BF16) attn_pooled_k<bf16_t, NJ><<<grid, 64, 0, s>>>(a); else attn_pooled_k<float, NJ><<<grid, 64, 0, s>>>(a); } while (0)
    if (hd <= 64) TP_ATTN_POOLED(1);
    else if (hd <= 128) TP_ATTN_POOLED(2);
    else if (hd <= 256) TP_ATTN_POOLED(4);
    else if (hd <= 512) TP_ATTN_POOLED(8);
    else TP_ATTN_POOLED(16);
#undef TP_ATTN_POOLED
    return tp_check_launch("attention (pooled, plain kernel)");
}

// ---- the mix over heads -----------------------------------------------------------------------------------------------
// a [rows, H, VG, hd] float32 (VG = KV: every head's weights on every kv head's values); out [rows, H, hd]:
// out_h = sum_g talk[h, g] a[g, kv(h)], the sum in float32 in the order of g.
template <typename T>
__global__ void __launch_bounds__(128)
talk_mix_k(const float* __restrict__ a, const float* __restrict__ talk, T* __restrict__ out, int H, int KV, int hd) {
    const int r = blockIdx.x, h = blockIdx.y, c = h / (H / KV);           // grid (rows, heads)
    const float* src = a + ((size_t)r * H * KV + c) * hd;                  // head g's sums on kv head c: + g KV hd
    for (int d = threadIdx.x; d < hd; d += 128) {
        float acc = 0.f;
        for (int g = 0; g < H; g++) acc = __builtin_fmaf(talk[h * H + g], src[(size_t)g * KV * hd + d], acc);
        st_f32(out + ((size_t)r * H + h) * hd + d, acc);
    }
}

extern "C" int tp_talk_mix(const float* a, const float* talk, void* out, int out_dtype, int M, int H, int KV, int hd, void* stream) {
    TP_REQUIRE(M > 0 && H > 0 && KV > 0 && hd > 0 && H % KV == 0, "talk_mix: shape rows=%d heads=%d kv=%d head_dim=%d", M, H, KV, hd);
    TP_REQUIRE(a && talk && out, "talk_mix: null operand");
    TP_REQUIRE(H <= 65535, "talk_mix: %d heads exceed one launch", H);
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == TP_BF16) talk_mix_k<bf16_t><<<dim3(M, H), 128, 0, s>>>(a, talk, (bf16_t*)out, H, KV, hd);
    else if (out_dtype == TP_F32) talk_mix_k<float><<<dim3(M, H), 128, 0, s>>>(a, talk, (float*)out, H, KV, hd);
    else return tp_fail("talk_mix: unknown dtype %d", out_dtype);
    return tp_check_launch("talk_mix");
}
