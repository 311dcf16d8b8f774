// Mixers that carry a matrix per head from token to token, and the small row-wise kernels around them.
//
//   shift_mix           out[s, r] = x[r] + (x[r - 1] - x[r]) * mu[s] within a sequence; the row before the step is a state
//   unary               x <- tanh(x) in place
//   time_mix_scan       o_t = (S + diag(u) k_t v_t^T)^T r_t;  S <- diag(w_t) S + k_t v_t^T,  w_t = exp(-exp(a_t + w0))
//   matrix_memory_scan  m' = max(f + m, i);  S <- e^(f + m - m') S + e^(i - m') k v^T, n likewise with k;
//                       o = S^T q / (max(|n . q|, e^(-m')) + 1e-6), i and f capped by a tanh
//   head_norm_gate      every head's part of a row over its root mean square, times a gain, times sigmoid(g) or silu(g)
//   weighted_sum        out = wa a + wb b
//
// Both scans run one wave for every (sequence, head, 64 value columns): a lane keeps one column of S in registers (all
// key rows), the per-row vectors of a token (k, q or r, the decay) live one row a lane and reach the others through
// lane reads, and the tokens of a sequence are taken in order, the next few tokens' loads in flight while the present
// ones are worked on.  States, gates, decays and sums are float32; nothing is added across waves.
#include "common.h"

__device__ __forceinline__ float lane_value(float x, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), lane));
}

enum { TP_GATE_SIGMOID = 0, TP_GATE_SILU = 1 };
#define TP_SCAN_AHEAD 4          // tokens whose loads are issued together

// ---- the mixes of a row with the row before it -----------------------------------------------------------------------
// grid (rows, blocks of 256 channels).  state [slots, D] float32: the last row of the sequence's step before.
template <typename T>
__global__ void __launch_bounds__(256)
shift_mix_k(const T* __restrict__ x, const float* __restrict__ mu, float* __restrict__ state, const int* __restrict__ slot_ids,
            const int* __restrict__ cu_rows, const int* __restrict__ row_seq, T* __restrict__ out, int M, int D, int n_mix, int save) {
    const int r = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= D) return;
    const int seq = row_seq[r];
    const bool first = r == cu_rows[seq];
    float* st = state + (size_t)slot_ids[seq] * D + c;
    const float cur = ld_f32(x + (size_t)r * D + c);
    const float before = first ? *st : ld_f32(x + (size_t)(r - 1) * D + c);
    const float diff = before - cur;
    for (int s = 0; s < n_mix; s++) st_f32(out + ((size_t)s * M + r) * D + c, __builtin_fmaf(diff, mu[(size_t)s * D + c], cur));
    if (save) *st = cur;                                  // every sequence brings one row: the same thread read it above
}

template <typename T>
__global__ void __launch_bounds__(256)
shift_save_k(const T* __restrict__ x, float* __restrict__ state, const int* __restrict__ slot_ids, const int* __restrict__ cu_rows, int D) {
    const int seq = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= D) return;
    state[(size_t)slot_ids[seq] * D + c] = ld_f32(x + (size_t)(cu_rows[seq + 1] - 1) * D + c);
}

extern "C" int tp_shift_mix(const void* x, int dtype, const float* mu, int n_mix, float* state, const int* slot_ids, const int* cu_rows,
                            const int* row_seq, void* out, int M, int n_seq, int D, int one_row_each, void* stream) {
    TP_REQUIRE(M > 0 && n_seq > 0 && D > 0 && n_mix > 0, "shift_mix: empty shape rows=%d sequences=%d channels=%d mixes=%d", M, n_seq, D, n_mix);
    TP_REQUIRE(x && mu && state && slot_ids && cu_rows && row_seq && out, "shift_mix: null operand");
    TP_REQUIRE(!one_row_each || M == n_seq, "shift_mix: one row each, but %d rows of %d sequences", M, n_seq);
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(M, tp_cdiv(D, 256)), grid_save(n_seq, tp_cdiv(D, 256));
    if (dtype == TP_BF16) {
        shift_mix_k<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)x, mu, state, slot_ids, cu_rows, row_seq, (bf16_t*)out, M, D, n_mix, one_row_each);
        if (!one_row_each) shift_save_k<bf16_t><<<grid_save, 256, 0, s>>>((const bf16_t*)x, state, slot_ids, cu_rows, D);
    } else if (dtype == TP_F32) {
        shift_mix_k<float><<<grid, 256, 0, s>>>((const float*)x, mu, state, slot_ids, cu_rows, row_seq, (float*)out, M, D, n_mix, one_row_each);
        if (!one_row_each) shift_save_k<float><<<grid_save, 256, 0, s>>>((const float*)x, state, slot_ids, cu_rows, D);
    } else return tp_fail("shift_mix: unknown dtype %d", dtype);
    return tp_check_launch("shift_mix");
}

// ---- x <- tanh(x) -------------------------------------------------------------------------------------------------------
template <typename T>
__global__ void unary_tanh_k(T* __restrict__ x, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < total) st_f32(x + i, tanhf(ld_f32(x + i)));
}

extern "C" int tp_unary_tanh(void* x, int dtype, long total, void* stream) {
    TP_REQUIRE(x && total > 0, "unary: empty tensor");
    const long blocks = (total + 255) / 256;
    TP_REQUIRE(blocks <= 0x7fffffffL, "unary: %ld elements exceed one launch", total);
    if (dtype == TP_BF16) unary_tanh_k<bf16_t><<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((bf16_t*)x, total);
    else if (dtype == TP_F32) unary_tanh_k<float><<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((float*)x, total);
    else return tp_fail("unary: unknown dtype %d", dtype);
    return tp_check_launch("unary");
}

// ---- out = wa a + wb b --------------------------------------------------------------------------------------------------
template <typename T>
__global__ void weighted_sum_k(const T* __restrict__ a, float wa, const T* __restrict__ b, float wb, float* __restrict__ out, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < total) out[i] = wa * ld_f32(a + i) + wb * ld_f32(b + i);
}

extern "C" int tp_weighted_sum(const void* a, float wa, const void* b, float wb, int dtype, float* out, long total, void* stream) {
    TP_REQUIRE(a && b && out && total > 0, "weighted_sum: empty or null operand");
    const long blocks = (total + 255) / 256;
    TP_REQUIRE(blocks <= 0x7fffffffL, "weighted_sum: %ld elements exceed one launch", total);
    if (dtype == TP_BF16) weighted_sum_k<bf16_t><<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((const bf16_t*)a, wa, (const bf16_t*)b, wb, out, total);
    else if (dtype == TP_F32) weighted_sum_k<float><<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((const float*)a, wa, (const float*)b, wb, out, total);
    else return tp_fail("weighted_sum: unknown dtype %d", dtype);
    return tp_check_launch("weighted_sum");
}

// ---- every head's part of a row over its root mean square, times gain and gate -----------------------------------------------
// grid (rows, heads), one wave each.  y float32 [M, H hs] contiguous; g [M, H hs] with a row stride.
template <typename TG, typename TO>
__global__ void __launch_bounds__(64)
head_norm_gate_k(const float* __restrict__ y, const float* __restrict__ gain, const TG* __restrict__ g, long g_stride, float eps,
                 TO* __restrict__ out, int H, int hs, int act) {
    const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* yr = y + ((size_t)r * H + h) * hs;
    float ss = 0.f;
    for (int d = lane; d < hs; d += 64) { const float v = yr[d]; ss = __builtin_fmaf(v, v, ss); }
    ss = wave_sum(ss);
    const float inv = rsqrtf(ss / (float)hs + eps);
    for (int d = lane; d < hs; d += 64) {
        const float gv = ld_f32(g + (size_t)r * g_stride + (size_t)h * hs + d);
        const float sg = 1.f / (1.f + expf(-gv));
        const float gate = act == TP_GATE_SILU ? gv * sg : sg;
        st_f32(out + ((size_t)r * H + h) * hs + d, (yr[d] * inv) * gain[(size_t)h * hs + d] * gate);
    }
}

extern "C" int tp_head_norm_gate(const float* y, const float* gain, const void* g, long g_stride, int g_dtype, float eps, void* out,
                                 int out_dtype, int M, int H, int hs, int act, void* stream) {
    TP_REQUIRE(M > 0 && H > 0 && hs > 0 && y && gain && g && out, "head_norm_gate: empty shape or null operand (M=%d H=%d size=%d)", M, H, hs);
    TP_REQUIRE(act == TP_GATE_SIGMOID || act == TP_GATE_SILU, "head_norm_gate: gate %d is neither sigmoid (%d) nor silu (%d)", act, TP_GATE_SIGMOID, TP_GATE_SILU);
    TP_REQUIRE(H <= 65535, "head_norm_gate: %d heads exceed one launch", H);
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(M, H);
    if (g_dtype == TP_BF16 && out_dtype == TP_BF16) head_norm_gate_k<bf16_t, bf16_t><<<grid, 64, 0, s>>>(y, gain, (const bf16_t*)g, g_stride, eps, (bf16_t*)out, H, hs, act);
    else if (g_dtype == TP_F32 && out_dtype == TP_F32) head_norm_gate_k<float, float><<<grid, 64, 0, s>>>(y, gain, (const float*)g, g_stride, eps, (float*)out, H, hs, act);
    else return tp_fail("head_norm_gate: gate dtype %d with output dtype %d has no kernel", g_dtype, out_dtype);
    return tp_check_launch("head_norm_gate");
}

// ---- the two scans ----------------------------------------------------------------------------------------------------------
// DK: key rows a lane keeps of its column (the head's key size rounded up to 16, 32 or a multiple of 64); NR registers
// hold a per-row vector, row (lane + 64 n) in register n.
template <typename T, int NR>
__device__ __forceinline__ void load_rows(float (&dst)[NR], const T* p, int rows, int lane, float scale) {
#pragma unroll
    for (int n = 0; n < NR; n++) {
        const int row = lane + 64 * n;
        dst[n] = row < rows ? ld_f32(p + row) * scale : 0.f;
    }
}

struct TimeMixArgs {
    const void* r; long r_stride; const void* k; long k_stride; const void* v; long v_stride;
    const float* log_rate; const float* w0; const float* bonus; float* state;
    const int* slot_ids; const int* cu_rows; float* y; int H, d;
};

template <typename T, int DK>
__global__ void __launch_bounds__(64)
time_mix_scan_k(TimeMixArgs a) {
    constexpr int NR = (DK + 63) / 64, AH = TP_SCAN_AHEAD;
    const int seq = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, j = blockIdx.z * 64 + lane;
    const int d = a.d, HD = a.H * d;
    const bool col = j < d;
    float* st = a.state + ((size_t)a.slot_ids[seq] * a.H + h) * d * d;
    float S[DK];
#pragma unroll
    for (int i = 0; i < DK; i++) S[i] = (col && i < d) ? st[(size_t)i * d + j] : 0.f;
    float u[NR], w0[NR];
    load_rows<float, NR>(u, a.bonus + (size_t)h * d, d, lane, 1.f);
    load_rows<float, NR>(w0, a.w0 + (size_t)h * d, d, lane, 1.f);
    const int begin = a.cu_rows[seq], end = a.cu_rows[seq + 1];
    float rr[AH][NR], kk[AH][NR], ww[AH][NR], vv[AH];
    auto fetch = [&](int t0, float (&R)[AH][NR], float (&K)[AH][NR], float (&W)[AH][NR], float (&V)[AH]) {
#pragma unroll
        for (int p = 0; p < AH; p++) {
            const int t = min(t0 + p, end - 1);          // past the end: a row that exists, never used
            load_rows<T, NR>(R[p], (const T*)a.r + (size_t)t * a.r_stride + (size_t)h * d, d, lane, 1.f);
            load_rows<T, NR>(K[p], (const T*)a.k + (size_t)t * a.k_stride + (size_t)h * d, d, lane, 1.f);
            load_rows<float, NR>(W[p], a.log_rate + (size_t)t * HD + (size_t)h * d, d, lane, 1.f);
            V[p] = col ? ld_f32((const T*)a.v + (size_t)t * a.v_stride + (size_t)h * d + j) : 0.f;
        }
    };
    fetch(begin, rr, kk, ww, vv);
    for (int t0 = begin; t0 < end; t0 += AH) {
        float rn[AH][NR], kn[AH][NR], wn[AH][NR], vn[AH];
        fetch(t0 + AH, rn, kn, wn, vn);
#pragma unroll
        for (int p = 0; p < AH; p++) {
            if (t0 + p >= end) break;
            float dot = 0.f;
#pragma unroll
            for (int n = 0; n < NR; n++) {
                ww[p][n] = lane + 64 * n < d ? expf(-expf(ww[p][n] + w0[n])) : 0.f;
                dot = __builtin_fmaf(rr[p][n] * u[n], kk[p][n], dot);
            }
            const float vj = vv[p];
            float o = wave_sum(dot) * vj;                // the present token's bonus: sum_i r_i u_i k_i, times v_j
#pragma unroll
            for (int i = 0; i < DK; i++) {
                const float ri = lane_value(rr[p][i / 64], i % 64), ki = lane_value(kk[p][i / 64], i % 64), wi = lane_value(ww[p][i / 64], i % 64);
                o = __builtin_fmaf(ri, S[i], o);
                S[i] = __builtin_fmaf(wi, S[i], ki * vj);
            }
            if (col) a.y[(size_t)(t0 + p) * HD + (size_t)h * d + j] = o;
        }
#pragma unroll
        for (int p = 0; p < AH; p++) {
            vv[p] = vn[p];
#pragma unroll
            for (int n = 0; n < NR; n++) { rr[p][n] = rn[p][n]; kk[p][n] = kn[p][n]; ww[p][n] = wn[p][n]; }
        }
    }
    if (col)
#pragma unroll
        for (int i = 0; i < DK; i++) if (i < d) st[(size_t)i * d + j] = S[i];
}

struct MatrixMemoryArgs {
    const void* q; long q_stride; const void* k; long k_stride; const void* v; long v_stride;
    const float* gates; float cap, q_scale; float* memory; float* normalizer; float* maximum;
    const int* slot_ids; const int* cu_rows; float* y; int H, dk, dv;
};

__device__ __forceinline__ float log_sigmoid_f(float z) { return -(log1pf(expf(-fabsf(z))) + fmaxf(-z, 0.f)); }

// One block for a (sequence, head), a wave for every 64 value columns: every wave carries n and m along (they are the
// same in all), reads them before any wave writes them back, and the first wave stores them at the end.
template <typename T, int DK>
__global__ void __launch_bounds__(256)
matrix_memory_scan_k(MatrixMemoryArgs a) {
    constexpr int NR = (DK + 63) / 64, AH = TP_SCAN_AHEAD;
    const int seq = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, j = threadIdx.x;
    const int dk = a.dk, dv = a.dv, H = a.H;
    const bool col = j < dv;
    const size_t slot = (size_t)a.slot_ids[seq];
    float* st = a.memory + (slot * H + h) * dk * dv;
    float* sn = a.normalizer + (slot * H + h) * dk;
    float S[DK], nn[NR];
#pragma unroll
    for (int i = 0; i < DK; i++) S[i] = (col && i < dk) ? st[(size_t)i * dv + j] : 0.f;
    load_rows<float, NR>(nn, sn, dk, lane, 1.f);
    float m = a.maximum[slot * H + h];
    __syncthreads();
    const int begin = a.cu_rows[seq], end = a.cu_rows[seq + 1];
    // lane p of a group of tokens forms token p's two gates; the others read them from it
    float qq[AH][NR], kk[AH][NR], vv[AH], gi, gf;
    auto fetch = [&](int t0, float (&Q)[AH][NR], float (&K)[AH][NR], float (&V)[AH], float& I, float& F) {
#pragma unroll
        for (int p = 0; p < AH; p++) {
            const int t = min(t0 + p, end - 1);
            load_rows<T, NR>(Q[p], (const T*)a.q + (size_t)t * a.q_stride + (size_t)h * dk, dk, lane, a.q_scale);
            load_rows<T, NR>(K[p], (const T*)a.k + (size_t)t * a.k_stride + (size_t)h * dk, dk, lane, 1.f);
            V[p] = col ? ld_f32((const T*)a.v + (size_t)t * a.v_stride + (size_t)h * dv + j) : 0.f;
        }
        const int t = min(t0 + min(lane, AH - 1), end - 1);
        I = a.gates[(size_t)t * 2 * H + h];
        F = a.gates[(size_t)t * 2 * H + H + h];
    };
    fetch(begin, qq, kk, vv, gi, gf);
    for (int t0 = begin; t0 < end; t0 += AH) {
        float qn[AH][NR], kn[AH][NR], vn[AH], gin, gfn;
        fetch(t0 + AH, qn, kn, vn, gin, gfn);
        const float li = a.cap * tanhf(gi / a.cap), lf = log_sigmoid_f(a.cap * tanhf(gf / a.cap));
#pragma unroll
        for (int p = 0; p < AH; p++) {
            if (t0 + p >= end) break;
            const float i_t = lane_value(li, p), f_t = lane_value(lf, p);
            const float m_new = fmaxf(f_t + m, i_t);
            const float keep = expf(f_t + m - m_new), take = expf(i_t - m_new);
            m = m_new;
            float dot = 0.f;
#pragma unroll
            for (int n = 0; n < NR; n++) {
                nn[n] = __builtin_fmaf(keep, nn[n], take * kk[p][n]);
                dot = __builtin_fmaf(nn[n], qq[p][n], dot);
            }
            const float den = fmaxf(fabsf(wave_sum(dot)), expf(-m)) + 1e-6f;
            const float tv = take * vv[p];
            float o = 0.f;
#pragma unroll
            for (int i = 0; i < DK; i++) {
                const float qi = lane_value(qq[p][i / 64], i % 64), ki = lane_value(kk[p][i / 64], i % 64);
                S[i] = __builtin_fmaf(keep, S[i], ki * tv);
                o = __builtin_fmaf(qi, S[i], o);
            }
            if (col) a.y[((size_t)(t0 + p) * H + h) * dv + j] = o / den;
        }
        gi = gin; gf = gfn;
#pragma unroll
        for (int p = 0; p < AH; p++) {
            vv[p] = vn[p];
#pragma unroll
            for (int n = 0; n < NR; n++) { qq[p][n] = qn[p][n]; kk[p][n] = kn[p][n]; }
        }
    }
    if (col)
#pragma unroll
        for (int i = 0; i < DK; i++) if (i < dk) st[(size_t)i * dv + j] = S[i];
    if (wave == 0) {
#pragma unroll
        for (int n = 0; n < NR; n++) if (lane + 64 * n < dk) sn[lane + 64 * n] = nn[n];
        if (lane == 0) a.maximum[slot * H + h] = m;
    }
}

#define TP_SCAN_SIZES(LAUNCH, rows) do { \
    if ((rows) <= 16) LAUNCH(16); else if ((rows) <= 32) LAUNCH(32); else if ((rows) <= 64) LAUNCH(64); \
    else if ((rows) <= 128) LAUNCH(128); else LAUNCH(256); } while (0)

// state [slots, H, d, d] float32 (key row, value column); log_rate float32 [M, H d] contiguous; y float32 [M, H d]
extern "C" int tp_time_mix_scan(const void* r, long r_stride, const void* k, long k_stride, const void* v, long v_stride, int dtype,
                                const float* log_rate, const float* w0, const float* bonus, float* state, const int* slot_ids,
                                const int* cu_rows, float* y, int n_seq, int H, int d, void* stream) {
    TP_REQUIRE(n_seq > 0 && H > 0 && d > 0, "time_mix_scan: empty shape sequences=%d heads=%d size=%d", n_seq, H, d);
    TP_REQUIRE(d <= 256, "time_mix_scan: heads of %d channels exceed the 256 a lane keeps", d);
    TP_REQUIRE(H <= 65535, "time_mix_scan: %d heads exceed one launch", H);
    TP_REQUIRE(r && k && v && log_rate && w0 && bonus && state && slot_ids && cu_rows && y, "time_mix_scan: null operand");
    TimeMixArgs a{r, r_stride, k, k_stride, v, v_stride, log_rate, w0, bonus, state, slot_ids, cu_rows, y, H, d};
    dim3 grid(n_seq, H, tp_cdiv(d, 64));
    hipStream_t s = (hipStream_t)stream;
    if (dtype != TP_BF16 && dtype != TP_F32) return tp_fail("time_mix_scan: unknown dtype %d", dtype);
#define TP_LAUNCH(DK) do { if (dtype == TP_BF16) time_mix_scan_k<bf16_t, DK><<<grid, 64, 0, s>>>(a); else time_mix_scan_k<float, DK><<<grid, 64, 0, s>>>(a); } while (0)
    TP_SCAN_SIZES(TP_LAUNCH, d);
#undef TP_LAUNCH
    return tp_check_launch("time_mix_scan");
}

// memory [slots, H, dk, dv], normalizer [slots, H, dk], maximum [slots, H], gates [M, 2 H] (input sums, then forget sums), all float32
extern "C" int tp_matrix_memory_scan(const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride, int dtype,
                                     const float* gates, float cap, float q_scale, float* memory, float* normalizer, float* maximum,
                                     const int* slot_ids, const int* cu_rows, float* y, int n_seq, int H, int dk, int dv, void* stream) {
    TP_REQUIRE(n_seq > 0 && H > 0 && dk > 0 && dv > 0, "matrix_memory_scan: empty shape sequences=%d heads=%d key=%d value=%d", n_seq, H, dk, dv);
    TP_REQUIRE(dk <= 256, "matrix_memory_scan: keys of %d elements exceed the 256 a lane keeps", dk);
    TP_REQUIRE(dv <= 256, "matrix_memory_scan: values of %d elements exceed the 256 columns of a block", dv);
    TP_REQUIRE(H <= 65535, "matrix_memory_scan: %d heads exceed one launch", H);
    TP_REQUIRE(cap > 0.f, "matrix_memory_scan: the gates' cap must be positive");
    TP_REQUIRE(q && k && v && gates && memory && normalizer && maximum && slot_ids && cu_rows && y, "matrix_memory_scan: null operand");
    MatrixMemoryArgs a{q, q_stride, k, k_stride, v, v_stride, gates, cap, q_scale, memory, normalizer, maximum, slot_ids, cu_rows, y, H, dk, dv};
    dim3 grid(n_seq, H);
    const int threads = 64 * tp_cdiv(dv, 64);
    hipStream_t s = (hipStream_t)stream;
    if (dtype != TP_BF16 && dtype != TP_F32) return tp_fail("matrix_memory_scan: unknown dtype %d", dtype);
#define TP_LAUNCH(DK) do { if (dtype == TP_BF16) matrix_memory_scan_k<bf16_t, DK><<<grid, threads, 0, s>>>(a); else matrix_memory_scan_k<float, DK><<<grid, threads, 0, s>>>(a); } while (0)
    TP_SCAN_SIZES(TP_LAUNCH, dk);
#undef TP_LAUNCH
    return tp_check_launch("matrix_memory_scan");
}
