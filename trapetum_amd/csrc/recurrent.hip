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
// Both scans give 64 value columns of a (sequence, head) to one wave, or, for heads of 64 key rows and more, to a few waves
// of a block that each keep a part of the rows: a lane keeps its wave's rows of one column of S in registers.  The per-row
// vectors of a token (k, q or r, the decay) are formed one row a lane by the block's first wave and reach all lanes through
// LDS, where every lane reads the same four rows at a time (lane reads into scalar registers cost more: a token's few
// hundred of them do not fit the scalar file).  The tokens of a sequence are taken in order, the next few tokens' loads in flight while the
// present ones are worked on; a row of S goes on by itself, an output is a sum over rows whose parts meet in LDS once for
// the tokens in flight.  States, gates, decays and sums are float32.
#include "common.h"

__device__ __forceinline__ float lane_value(float x, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), lane));
}

enum { TP_GATE_SIGMOID = 0, TP_GATE_SILU = 1 };
#define TP_SCAN_AHEAD 4          // tokens whose loads are issued together

// ---- the mixes of a row with the row before it -----------------------------------------------------------------------
// grid (rows, blocks of 256 channels).  state [slots, D] float32: the last row of the sequence's step before.
template <typename T, typename TO>
__global__ void __launch_bounds__(256)
shift_mix_k(const T* __restrict__ x, const float* __restrict__ mu, float* __restrict__ state, const int* __restrict__ slot_ids,
            const int* __restrict__ cu_rows, const int* __restrict__ row_seq, TO* __restrict__ out, int M, int D, int n_mix, int save) {
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

// out_dtype: the mixes' dtype; it may be narrower than the rows' (float32 rows of a norm, mixes in bfloat16: one rounding)
extern "C" int tp_shift_mix(const void* x, int dtype, const float* mu, int n_mix, float* state, const int* slot_ids, const int* cu_rows,
                            const int* row_seq, void* out, int out_dtype, int M, int n_seq, int D, int one_row_each, void* stream) {
    TP_REQUIRE(M > 0 && n_seq > 0 && D > 0 && n_mix > 0, "shift_mix: empty shape rows=%d sequences=%d channels=%d mixes=%d", M, n_seq, D, n_mix);
    TP_REQUIRE(x && mu && state && slot_ids && cu_rows && row_seq && out, "shift_mix: null operand");
    TP_REQUIRE(!one_row_each || M == n_seq, "shift_mix: one row each, but %d rows of %d sequences", M, n_seq);
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(M, tp_cdiv(D, 256)), grid_save(n_seq, tp_cdiv(D, 256));
    if (dtype == TP_BF16 && out_dtype == TP_BF16) {
        shift_mix_k<bf16_t, bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)x, mu, state, slot_ids, cu_rows, row_seq, (bf16_t*)out, M, D, n_mix, one_row_each);
        if (!one_row_each) shift_save_k<bf16_t><<<grid_save, 256, 0, s>>>((const bf16_t*)x, state, slot_ids, cu_rows, D);
    } else if (dtype == TP_F32 && (out_dtype == TP_F32 || out_dtype == TP_BF16)) {
        if (out_dtype == TP_F32) shift_mix_k<float, float><<<grid, 256, 0, s>>>((const float*)x, mu, state, slot_ids, cu_rows, row_seq, (float*)out, M, D, n_mix, one_row_each);
        else shift_mix_k<float, bf16_t><<<grid, 256, 0, s>>>((const float*)x, mu, state, slot_ids, cu_rows, row_seq, (bf16_t*)out, M, D, n_mix, one_row_each);
        if (!one_row_each) shift_save_k<float><<<grid_save, 256, 0, s>>>((const float*)x, state, slot_ids, cu_rows, D);
    } else return tp_fail("shift_mix: no kernel from dtype %d to dtype %d", dtype, out_dtype);
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

// A long sequence is cut into chunks of `chunk` rows that run side by side (MODE): 1, every chunk but a sequence's last from
// a zero state and without outputs, leaving what the chunk adds to the state and the decay over the chunk in a workspace;
// then a carry kernel walks a sequence's chunks in order and leaves every chunk's true first state there; 2, every chunk
// again from that state, with outputs, the last one leaving the sequence's state in its slot.  MODE 0 is the whole
// sequence in one wave, from and to the slot.  The arithmetic of a row is the same in all three.
enum { TP_SCAN_WHOLE = 0, TP_SCAN_LOCAL = 1, TP_SCAN_FINAL = 2 };

struct TimeMixArgs {
    const void* r; long r_stride; const void* k; long k_stride; const void* v; long v_stride;
    const float* log_rate; const float* w0; const float* bonus; float* state;
    const int* slot_ids; const int* cu_rows; float* y; int H, d;
    int chunk, n_chunks; float* ws_state; float* ws_decay;      // [sequences n_chunks, H, d, d] and [sequences n_chunks, H, d]
};

// Key rows of a head that one wave keeps: heads of 64 rows and more are split over four waves of a block (a row of S
// goes on by itself; only an output is a sum over rows, and the waves' parts of it meet in LDS once for the tokens in
// flight), so that a state is read by four times the waves and a lane keeps a quarter of a column.
#define TP_SCAN_SPLIT(DK) ((DK) >= 64 ? 4 : 1)

template <typename T, int DK, int MODE>
__global__ void __launch_bounds__(64 * TP_SCAN_SPLIT(DK))
time_mix_scan_k(TimeMixArgs a) {
    constexpr int NR = (DK + 63) / 64, AH = TP_SCAN_AHEAD, RS = TP_SCAN_SPLIT(DK), DKW = DK / RS;
    const int h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, j = blockIdx.z * 64 + lane, row0 = wave * DKW;
    const int seq = MODE == TP_SCAN_WHOLE ? blockIdx.x : blockIdx.x / a.n_chunks;
    const int d = a.d, HD = a.H * d;
    const bool col = j < d;
    int begin = a.cu_rows[seq], end = a.cu_rows[seq + 1];
    bool last = true;
    if (MODE != TP_SCAN_WHOLE) {
        begin += (blockIdx.x % a.n_chunks) * a.chunk;
        if (begin >= end) return;
        last = begin + a.chunk >= end;
        if (MODE == TP_SCAN_LOCAL && last) return;           // nothing comes after it
        end = min(end, begin + a.chunk);
    }
    float* st = a.state + ((size_t)a.slot_ids[seq] * a.H + h) * d * d;
    float* wst = MODE == TP_SCAN_WHOLE ? st : a.ws_state + ((size_t)blockIdx.x * a.H + h) * d * d;
    const float* from = MODE == TP_SCAN_FINAL ? wst : st;
    float S[DKW];                                       // rows row0 .. row0 + DKW - 1 of column j
#pragma unroll
    for (int i = 0; i < DKW; i++) {                     // every lane reads an element that exists; what is none of S becomes zero
        const float x = MODE != TP_SCAN_LOCAL ? from[min(row0 + i, d - 1) * d + min(j, d - 1)] : 0.f;
        S[i] = (col && row0 + i < d) ? x : 0.f;
    }
    float u[NR], w0[NR], fall[NR];                       // fall: the sum of the rows' log decays over the chunk
    load_rows<float, NR>(u, a.bonus + (size_t)h * d, d, lane, 1.f);
    load_rows<float, NR>(w0, a.w0 + (size_t)h * d, d, lane, 1.f);
#pragma unroll
    for (int n = 0; n < NR; n++) fall[n] = 0.f;
    // the block's first wave forms the per-row vectors of the tokens in flight for all its waves
    const bool stager = RS == 1 || wave == 0;
    float rr[AH][NR] = {}, kk[AH][NR] = {}, ww[AH][NR] = {}, vv[AH];
    auto fetch = [&](int t0, float (&R)[AH][NR], float (&K)[AH][NR], float (&W)[AH][NR], float (&V)[AH]) {
#pragma unroll
        for (int p = 0; p < AH; p++) {
            const int t = min(t0 + p, end - 1);          // past the end: a row that exists, never used
            if (stager) {
                if (MODE != TP_SCAN_LOCAL) load_rows<T, NR>(R[p], (const T*)a.r + (size_t)t * a.r_stride + (size_t)h * d, d, lane, 1.f);
                load_rows<T, NR>(K[p], (const T*)a.k + (size_t)t * a.k_stride + (size_t)h * d, d, lane, 1.f);
                load_rows<float, NR>(W[p], a.log_rate + (size_t)t * HD + (size_t)h * d, d, lane, 1.f);
            }
            V[p] = col ? ld_f32((const T*)a.v + (size_t)t * a.v_stride + (size_t)h * d + j) : 0.f;
        }
    };
    // the per-row vectors of the tokens in flight, written a row a lane and read back by every lane, four rows a read
    __shared__ __attribute__((aligned(16))) float stage_all[2][AH][3][DK];       // for rounds in turn
    __shared__ float parts[2][RS][AH][64];               // the waves' parts of the outputs, for rounds in turn
    int round = 0;
    fetch(begin, rr, kk, ww, vv);
    for (int t0 = begin; t0 < end; t0 += AH, round ^= 1) {
        float (*stage)[3][DK] = stage_all[round];
        float rn[AH][NR] = {}, kn[AH][NR] = {}, wn[AH][NR] = {}, vn[AH];
        fetch(t0 + AH, rn, kn, wn, vn);
        float bonus_dot[AH] = {};
        if (stager)
#pragma unroll
        for (int p = 0; p < AH; p++) {
            float dot = 0.f;
#pragma unroll
            for (int n = 0; n < NR; n++) {
                const int row = lane + 64 * n;
                const float lw = -expf(ww[p][n] + w0[n]);
                if (MODE == TP_SCAN_LOCAL && t0 + p < end) fall[n] += lw;
                if (MODE != TP_SCAN_LOCAL) dot = __builtin_fmaf(rr[p][n] * u[n], kk[p][n], dot);
                if (row < DK) {
                    if (MODE != TP_SCAN_LOCAL) stage[p][0][row] = rr[p][n];
                    stage[p][1][row] = kk[p][n];
                    stage[p][2][row] = row < d ? expf(lw) : 0.f;
                }
            }
            bonus_dot[p] = MODE != TP_SCAN_LOCAL ? wave_sum(dot) : 0.f;     // the present token's bonus: sum_i r_i u_i k_i
        }
        if (RS > 1) __syncthreads();
        else {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        float outs[AH];                                  // stored together after the tokens: no branch of the lanes between them
#pragma unroll
        for (int p = 0; p < AH; p++) {
            outs[p] = 0.f;
            if (t0 + p < end) {
                const float vj = vv[p];
                const float4* R4 = (const float4*)(stage[p][0] + row0);
                const float4* K4 = (const float4*)(stage[p][1] + row0);
                const float4* W4 = (const float4*)(stage[p][2] + row0);
                if (MODE == TP_SCAN_LOCAL) {
#pragma unroll
                    for (int i = 0; i < DKW; i += 4) {
                        if (i % 16 == 0) __builtin_amdgcn_sched_barrier(0);      // the reads of sixteen rows at a time, not of all
                        const float4 k4 = K4[i / 4], w4 = W4[i / 4];
                        S[i] = __builtin_fmaf(w4.x, S[i], k4.x * vj);
                        S[i + 1] = __builtin_fmaf(w4.y, S[i + 1], k4.y * vj);
                        S[i + 2] = __builtin_fmaf(w4.z, S[i + 2], k4.z * vj);
                        S[i + 3] = __builtin_fmaf(w4.w, S[i + 3], k4.w * vj);
                    }
                } else {
                    float o0 = wave == 0 ? bonus_dot[p] * vj : 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;       // four sums: no FMA waits for the one before
#pragma unroll
                    for (int i = 0; i < DKW; i += 4) {
                        if (i % 16 == 0) __builtin_amdgcn_sched_barrier(0);      // the reads of sixteen rows at a time, not of all
                        const float4 r4 = R4[i / 4], k4 = K4[i / 4], w4 = W4[i / 4];
                        o0 = __builtin_fmaf(r4.x, S[i], o0);
                        S[i] = __builtin_fmaf(w4.x, S[i], k4.x * vj);
                        o1 = __builtin_fmaf(r4.y, S[i + 1], o1);
                        S[i + 1] = __builtin_fmaf(w4.y, S[i + 1], k4.y * vj);
                        o2 = __builtin_fmaf(r4.z, S[i + 2], o2);
                        S[i + 2] = __builtin_fmaf(w4.z, S[i + 2], k4.z * vj);
                        o3 = __builtin_fmaf(r4.w, S[i + 3], o3);
                        S[i + 3] = __builtin_fmaf(w4.w, S[i + 3], k4.w * vj);
                    }
                    outs[p] = (o0 + o1) + (o2 + o3);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (MODE != TP_SCAN_LOCAL) {
            if (RS > 1) {                                // wave p adds the waves' parts of token p and stores it
                static_assert(RS == 1 || RS == AH, "a wave for every token in flight");
#pragma unroll
                for (int p = 0; p < AH; p++) parts[round][wave][p][lane] = outs[p];
                __syncthreads();
                float sum = 0.f;
#pragma unroll
                for (int w = 0; w < RS; w++) sum += parts[round][w][wave][lane];
                if (col && t0 + wave < end) a.y[(size_t)(t0 + wave) * HD + (size_t)h * d + j] = sum;
            } else if (col) {
#pragma unroll
                for (int p = 0; p < AH; p++) if (t0 + p < end) a.y[(size_t)(t0 + p) * HD + (size_t)h * d + j] = outs[p];
            }
        }
#pragma unroll
        for (int p = 0; p < AH; p++) {
            vv[p] = vn[p];
#pragma unroll
            for (int n = 0; n < NR; n++) { rr[p][n] = rn[p][n]; kk[p][n] = kn[p][n]; ww[p][n] = wn[p][n]; }
        }
    }
    float* to = MODE == TP_SCAN_LOCAL ? wst : st;
    if (col && (MODE != TP_SCAN_FINAL || last))
#pragma unroll
        for (int i = 0; i < DKW; i++) if (row0 + i < d) to[(row0 + i) * d + j] = S[i];
    if (MODE == TP_SCAN_LOCAL && blockIdx.z == 0 && wave == 0)
#pragma unroll
        for (int n = 0; n < NR; n++) if (lane + 64 * n < d) a.ws_decay[((size_t)blockIdx.x * a.H + h) * d + lane + 64 * n] = expf(fall[n]);
}

// Chunk after chunk of a sequence: the state a chunk starts from takes the place of what the chunk adds, and the next
// one is  decay * state + what it adds.  grid (sequences, heads, blocks of 256 elements of the state); the loads of
// eight chunks are in flight together.
__global__ void __launch_bounds__(256)
time_mix_carry_k(const float* __restrict__ state, const int* __restrict__ slot_ids, const int* __restrict__ cu_rows,
                 float* ws_state, const float* __restrict__ ws_decay, int H, int d, int chunk, int n_chunks) {
    const int seq = blockIdx.x, h = blockIdx.y, e = blockIdx.z * 256 + threadIdx.x;
    const int n = (cu_rows[seq + 1] - cu_rows[seq] + chunk - 1) / chunk;
    if (e >= d * d || n <= 0) return;
    const int i = e / d;
    float S = state[((size_t)slot_ids[seq] * H + h) * d * d + e];
    const size_t g0 = (size_t)seq * n_chunks;
    for (int c0 = 0; c0 < n; c0 += 8) {
        float L[8], D[8];
#pragma unroll
        for (int p = 0; p < 8; p++) {
            const int c = c0 + p;
            L[p] = c < n - 1 ? ws_state[((g0 + c) * H + h) * d * d + e] : 0.f;
            D[p] = c < n - 1 ? ws_decay[((g0 + c) * H + h) * d + i] : 0.f;
        }
#pragma unroll
        for (int p = 0; p < 8; p++) {
            const int c = c0 + p;
            if (c < n) ws_state[((g0 + c) * H + h) * d * d + e] = S;
            S = __builtin_fmaf(D[p], S, L[p]);
        }
    }
}

struct MatrixMemoryArgs {
    const void* q; long q_stride; const void* k; long k_stride; const void* v; long v_stride;
    const float* gates; float cap, q_scale; float* memory; float* normalizer; float* maximum;
    const int* slot_ids; const int* cu_rows; float* y; int H, dk, dv;
    // chunks as above.  ws_state [sequences n_chunks, H, dk dv + dk]: a chunk's matrix, then its normalizer, both in units
    // of e^(its maximum); ws_aux [sequences n_chunks, H, 4]: the maximum of a chunk run from nothing, the sum of its log
    // forget gates, the maximum it really starts from
    int chunk, n_chunks; float* ws_state; float* ws_aux;
};

__device__ __forceinline__ float log_sigmoid_f(float z) { return -(log1pf(expf(-fabsf(z))) + fmaxf(-z, 0.f)); }

// One block for a (sequence, head) or a (chunk, head), a group of waves for every 64 value columns: every wave carries n
// and m along (they are the same in all), reads them before any wave writes them back, and the first wave stores them at
// the end.  A chunk run from nothing starts with m = -inf: its first row's maximum is its input gate, and nothing is kept.
// The matrix memory's split: a block holds up to four groups of 64 value columns, each in MM_SPLIT waves
#define TP_MM_SPLIT(DK) ((DK) >= 256 ? 2 : (DK) >= 64 ? 4 : 1)

template <typename T, int DK, int MODE>
__global__ void __launch_bounds__(256 * TP_MM_SPLIT(DK))
matrix_memory_scan_k(MatrixMemoryArgs a) {
    constexpr int NR = (DK + 63) / 64, RS = TP_MM_SPLIT(DK), AH = RS > 1 ? 2 : TP_SCAN_AHEAD, DKW = DK / RS;
    const int h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, group = wave / RS, part = wave % RS;
    const int j = group * 64 + lane, row0 = part * DKW;
    const int seq = MODE == TP_SCAN_WHOLE ? blockIdx.x : blockIdx.x / a.n_chunks;
    const int dk = a.dk, dv = a.dv, H = a.H;
    const bool col = j < dv;
    int begin = a.cu_rows[seq], end = a.cu_rows[seq + 1];
    bool last = true;
    if (MODE != TP_SCAN_WHOLE) {
        begin += (blockIdx.x % a.n_chunks) * a.chunk;
        if (begin >= end) return;
        last = begin + a.chunk >= end;
        if (MODE == TP_SCAN_LOCAL && last) return;
        end = min(end, begin + a.chunk);
    }
    const size_t slot = (size_t)a.slot_ids[seq];
    float* st = a.memory + (slot * H + h) * dk * dv;
    float* sn = a.normalizer + (slot * H + h) * dk;
    float* wst = MODE == TP_SCAN_WHOLE ? st : a.ws_state + ((size_t)blockIdx.x * H + h) * ((size_t)dk * dv + dk);
    float* aux = MODE == TP_SCAN_WHOLE ? sn : a.ws_aux + ((size_t)blockIdx.x * H + h) * 4;
    const float* from = MODE == TP_SCAN_FINAL ? wst : st;
    float S[DKW], nn[NR];                               // rows row0 .. row0 + DKW - 1 of column j; all of n, a row a lane
#pragma unroll
    for (int i = 0; i < DKW; i++) {                     // every lane reads an element that exists; what is none of S becomes zero
        const float x = MODE != TP_SCAN_LOCAL ? from[min(row0 + i, dk - 1) * dv + min(j, dv - 1)] : 0.f;
        S[i] = (col && row0 + i < dk) ? x : 0.f;
    }
    float m = -INFINITY, fsum = 0.f;
    if (MODE == TP_SCAN_LOCAL) {
#pragma unroll
        for (int n = 0; n < NR; n++) nn[n] = 0.f;
    } else {
        load_rows<float, NR>(nn, MODE == TP_SCAN_FINAL ? wst + (size_t)dk * dv : sn, dk, lane, 1.f);
        m = MODE == TP_SCAN_FINAL ? aux[2] : a.maximum[slot * H + h];
    }
    __syncthreads();
    // lane p of a group of tokens forms token p's two gates; the others read them from it
    // the block's first wave forms q and k of the tokens in flight for all its waves, carries n and forms the denominators
    const bool stager = wave == 0;
    float qq[AH][NR] = {}, kk[AH][NR] = {}, vv[AH], gi, gf;
    auto fetch = [&](int t0, float (&Q)[AH][NR], float (&K)[AH][NR], float (&V)[AH], float& I, float& F) {
#pragma unroll
        for (int p = 0; p < AH; p++) {
            const int t = min(t0 + p, end - 1);
            if (stager) {
                if (MODE != TP_SCAN_LOCAL) load_rows<T, NR>(Q[p], (const T*)a.q + (size_t)t * a.q_stride + (size_t)h * dk, dk, lane, a.q_scale);
                load_rows<T, NR>(K[p], (const T*)a.k + (size_t)t * a.k_stride + (size_t)h * dk, dk, lane, 1.f);
            }
            V[p] = col ? ld_f32((const T*)a.v + (size_t)t * a.v_stride + (size_t)h * dv + j) : 0.f;
        }
        const int t = min(t0 + min(lane, AH - 1), end - 1);
        I = a.gates[(size_t)t * 2 * H + h];
        F = a.gates[(size_t)t * 2 * H + H + h];
    };
    // q and k of the tokens in flight, written a row a lane by the first wave and read back by every lane; for rounds in turn
    __shared__ __attribute__((aligned(16))) float stage_all[2][AH][2][DK];
    __shared__ float dens_all[2][AH];
    __shared__ float parts[2][4 * RS][AH][64];           // the waves' parts of the outputs, for rounds in turn
    int round = 0;
    fetch(begin, qq, kk, vv, gi, gf);
    for (int t0 = begin; t0 < end; t0 += AH, round ^= 1) {
        float (*stage)[2][DK] = stage_all[round];
        float qn[AH][NR] = {}, kn[AH][NR] = {}, vn[AH], gin, gfn;
        fetch(t0 + AH, qn, kn, vn, gin, gfn);
        const float li = a.cap * tanhf(gi / a.cap), lf = log_sigmoid_f(a.cap * tanhf(gf / a.cap));
        // what the gates make of m, token after token: every wave for itself
        float keeps[AH], takes[AH], floors[AH];
#pragma unroll
        for (int p = 0; p < AH; p++) {
            keeps[p] = 1.f; takes[p] = 0.f; floors[p] = 1.f;
            if (t0 + p < end) {
                const float i_t = lane_value(li, p), f_t = lane_value(lf, p);
                const float m_new = fmaxf(f_t + m, i_t);
                keeps[p] = expf(f_t + m - m_new);
                takes[p] = expf(i_t - m_new);
                m = m_new;
                floors[p] = expf(-m);
                if (MODE == TP_SCAN_LOCAL) fsum += f_t;
            }
        }
        if (stager)
#pragma unroll
            for (int p = 0; p < AH; p++) {
                float dot = 0.f;
#pragma unroll
                for (int n = 0; n < NR; n++) {
                    const int row = lane + 64 * n;
                    if (t0 + p < end) nn[n] = __builtin_fmaf(keeps[p], nn[n], takes[p] * kk[p][n]);
                    if (MODE != TP_SCAN_LOCAL) dot = __builtin_fmaf(nn[n], qq[p][n], dot);
                    if (row < DK) {
                        if (MODE != TP_SCAN_LOCAL) stage[p][0][row] = qq[p][n];
                        stage[p][1][row] = kk[p][n];
                    }
                }
                if (MODE != TP_SCAN_LOCAL) {
                    const float den = fmaxf(fabsf(wave_sum(dot)), floors[p]) + 1e-6f;
                    if (lane == 0) dens_all[round][p] = den;
                }
            }
        __syncthreads();
        float outs[AH], dens[AH];                        // stored together after the tokens: no branch of the lanes between them
#pragma unroll
        for (int p = 0; p < AH; p++) {
            outs[p] = 0.f;
            dens[p] = MODE != TP_SCAN_LOCAL ? dens_all[round][p] : 1.f;
            if (t0 + p < end) {
                const float keep = keeps[p];
                const float tv = takes[p] * vv[p];
                const float4* Q4 = (const float4*)(stage[p][0] + row0);
                const float4* K4 = (const float4*)(stage[p][1] + row0);
                if (MODE == TP_SCAN_LOCAL) {
#pragma unroll
                    for (int i = 0; i < DKW; i += 4) {
                        if (i % 16 == 0) __builtin_amdgcn_sched_barrier(0);      // the reads of sixteen rows at a time, not of all
                        const float4 k4 = K4[i / 4];
                        S[i] = __builtin_fmaf(keep, S[i], k4.x * tv);
                        S[i + 1] = __builtin_fmaf(keep, S[i + 1], k4.y * tv);
                        S[i + 2] = __builtin_fmaf(keep, S[i + 2], k4.z * tv);
                        S[i + 3] = __builtin_fmaf(keep, S[i + 3], k4.w * tv);
                    }
                } else {
                    float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;                    // four sums: no FMA waits for the one before
#pragma unroll
                    for (int i = 0; i < DKW; i += 4) {
                        if (i % 16 == 0) __builtin_amdgcn_sched_barrier(0);      // the reads of sixteen rows at a time, not of all
                        const float4 q4 = Q4[i / 4], k4 = K4[i / 4];
                        S[i] = __builtin_fmaf(keep, S[i], k4.x * tv);
                        o0 = __builtin_fmaf(q4.x, S[i], o0);
                        S[i + 1] = __builtin_fmaf(keep, S[i + 1], k4.y * tv);
                        o1 = __builtin_fmaf(q4.y, S[i + 1], o1);
                        S[i + 2] = __builtin_fmaf(keep, S[i + 2], k4.z * tv);
                        o2 = __builtin_fmaf(q4.z, S[i + 2], o2);
                        S[i + 3] = __builtin_fmaf(keep, S[i + 3], k4.w * tv);
                        o3 = __builtin_fmaf(q4.w, S[i + 3], o3);
                    }
                    outs[p] = (o0 + o1) + (o2 + o3);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (MODE != TP_SCAN_LOCAL) {
            if (RS > 1) {                                // a group's first wave adds the parts of its waves
#pragma unroll
                for (int p = 0; p < AH; p++) parts[round][wave][p][lane] = outs[p];
                __syncthreads();
                if (part == 0)
#pragma unroll
                    for (int p = 0; p < AH; p++) {
                        float sum = 0.f;
#pragma unroll
                        for (int w = 0; w < RS; w++) sum += parts[round][group * RS + w][p][lane];
                        outs[p] = sum;
                    }
            }
            if (col && part == 0)
#pragma unroll
                for (int p = 0; p < AH; p++) if (t0 + p < end) a.y[((size_t)(t0 + p) * H + h) * dv + j] = outs[p] / dens[p];
        }
        gi = gin; gf = gfn;
#pragma unroll
        for (int p = 0; p < AH; p++) {
            vv[p] = vn[p];
#pragma unroll
            for (int n = 0; n < NR; n++) { qq[p][n] = qn[p][n]; kk[p][n] = kn[p][n]; }
        }
    }
    if (MODE == TP_SCAN_FINAL && !last) return;
    float* to = MODE == TP_SCAN_LOCAL ? wst : st;
    float* to_n = MODE == TP_SCAN_LOCAL ? wst + (size_t)dk * dv : sn;
    if (col)
#pragma unroll
        for (int i = 0; i < DKW; i++) if (row0 + i < dk) to[(row0 + i) * dv + j] = S[i];
    if (wave == 0) {
#pragma unroll
        for (int n = 0; n < NR; n++) if (lane + 64 * n < dk) to_n[lane + 64 * n] = nn[n];
        if (lane == 0) {
            if (MODE == TP_SCAN_LOCAL) { aux[0] = m; aux[1] = fsum; }
            else a.maximum[slot * H + h] = m;
        }
    }
}

// As time_mix_carry_k, over the dk dv elements of the matrix and the dk of the normalizer; with F a chunk's summed log
// forget gates and M the maximum it reaches from nothing, a state x in units of e^m goes on as
// m' = max(F + m, M), x' = e^(F + m - m') x + e^(M - m') (what the chunk adds).
__global__ void __launch_bounds__(256)
matrix_memory_carry_k(const float* __restrict__ memory, const float* __restrict__ normalizer, const float* __restrict__ maximum,
                      const int* __restrict__ slot_ids, const int* __restrict__ cu_rows, float* ws_state, float* ws_aux,
                      int H, int dk, int dv, int chunk, int n_chunks) {
    const int seq = blockIdx.x, h = blockIdx.y, e = blockIdx.z * 256 + threadIdx.x;
    const int n = (cu_rows[seq + 1] - cu_rows[seq] + chunk - 1) / chunk;
    const int per = dk * dv + dk;
    if (e >= per || n <= 0) return;
    const size_t slot = (size_t)slot_ids[seq];
    float x = e < dk * dv ? memory[(slot * H + h) * dk * dv + e] : normalizer[(slot * H + h) * dk + e - dk * dv];
    float m = maximum[slot * H + h];
    const size_t g0 = (size_t)seq * n_chunks;
    for (int c0 = 0; c0 < n; c0 += 8) {
        float L[8], M[8], F[8];
#pragma unroll
        for (int p = 0; p < 8; p++) {
            const int c = c0 + p;
            const bool next = c < n - 1;
            L[p] = next ? ws_state[((g0 + c) * H + h) * per + e] : 0.f;
            M[p] = next ? ws_aux[((g0 + c) * H + h) * 4] : 0.f;
            F[p] = next ? ws_aux[((g0 + c) * H + h) * 4 + 1] : 0.f;
        }
#pragma unroll
        for (int p = 0; p < 8; p++) {
            const int c = c0 + p;
            if (c < n) {
                ws_state[((g0 + c) * H + h) * per + e] = x;
                if (e == 0) ws_aux[((g0 + c) * H + h) * 4 + 2] = m;
            }
            const float m_new = fmaxf(F[p] + m, M[p]);
            x = __builtin_fmaf(expf(F[p] + m - m_new), x, expf(M[p] - m_new) * L[p]);
            m = m_new;
        }
    }
}

#define TP_SCAN_SIZES(LAUNCH, rows) do { \
    if ((rows) <= 16) LAUNCH(16); else if ((rows) <= 32) LAUNCH(32); else if ((rows) <= 64) LAUNCH(64); \
    else if ((rows) <= 128) LAUNCH(128); else LAUNCH(256); } while (0)

// The launches of a scan: whole sequences (chunk 0), or chunks of `chunk` rows (n_chunks of them cover the longest sequence).
#define TP_SCAN_MODES(KERNEL, CARRY, DK, whole_grid, chunk_grid, threads) do { \
    if (chunk <= 0) { \
        if (dtype == TP_BF16) KERNEL<bf16_t, DK, TP_SCAN_WHOLE><<<whole_grid, threads, 0, s>>>(a); \
        else KERNEL<float, DK, TP_SCAN_WHOLE><<<whole_grid, threads, 0, s>>>(a); \
    } else { \
        if (n_chunks > 1) { \
            if (dtype == TP_BF16) KERNEL<bf16_t, DK, TP_SCAN_LOCAL><<<chunk_grid, threads, 0, s>>>(a); \
            else KERNEL<float, DK, TP_SCAN_LOCAL><<<chunk_grid, threads, 0, s>>>(a); \
        } \
        CARRY; \
        if (dtype == TP_BF16) KERNEL<bf16_t, DK, TP_SCAN_FINAL><<<chunk_grid, threads, 0, s>>>(a); \
        else KERNEL<float, DK, TP_SCAN_FINAL><<<chunk_grid, threads, 0, s>>>(a); \
    } } while (0)

extern "C" long tp_time_mix_scan_workspace_floats(int n_seq, int n_chunks, int H, int d) {
    return (long)n_seq * n_chunks * H * ((long)d * d + d);
}

// state [slots, H, d, d] float32 (key row, value column); log_rate float32 [M, H d] contiguous; y float32 [M, H d].
// chunk > 0: sequences run in chunks of that many rows, n_chunks covering the longest; workspace: floats as above
extern "C" int tp_time_mix_scan(const void* r, long r_stride, const void* k, long k_stride, const void* v, long v_stride, int dtype,
                                const float* log_rate, const float* w0, const float* bonus, float* state, const int* slot_ids,
                                const int* cu_rows, float* y, int n_seq, int H, int d, int chunk, int n_chunks, float* workspace,
                                void* stream) {
    TP_REQUIRE(n_seq > 0 && H > 0 && d > 0, "time_mix_scan: empty shape sequences=%d heads=%d size=%d", n_seq, H, d);
    TP_REQUIRE(d <= 256, "time_mix_scan: heads of %d channels exceed the 256 a lane keeps", d);
    TP_REQUIRE(H <= 65535, "time_mix_scan: %d heads exceed one launch", H);
    TP_REQUIRE(r && k && v && log_rate && w0 && bonus && state && slot_ids && cu_rows && y, "time_mix_scan: null operand");
    TP_REQUIRE(chunk == 0 || (chunk > 0 && n_chunks > 0 && workspace && (long)n_seq * n_chunks <= 0x7fffffffL),
               "time_mix_scan: %d chunks of %d rows need a workspace", n_chunks, chunk);
    float* ws_decay = workspace ? workspace + (size_t)n_seq * n_chunks * H * d * d : nullptr;
    TimeMixArgs a{r, r_stride, k, k_stride, v, v_stride, log_rate, w0, bonus, state, slot_ids, cu_rows, y, H, d,
                  chunk, n_chunks, workspace, ws_decay};
    dim3 grid(n_seq, H, tp_cdiv(d, 64)), chunk_grid(n_seq * (chunk > 0 ? n_chunks : 1), H, tp_cdiv(d, 64)), carry_grid(n_seq, H, tp_cdiv(d * d, 256));
    hipStream_t s = (hipStream_t)stream;
    if (dtype != TP_BF16 && dtype != TP_F32) return tp_fail("time_mix_scan: unknown dtype %d", dtype);
#define TP_LAUNCH(DK) TP_SCAN_MODES(time_mix_scan_k, (time_mix_carry_k<<<carry_grid, 256, 0, s>>>(state, slot_ids, cu_rows, workspace, ws_decay, H, d, chunk, n_chunks)), DK, grid, chunk_grid, 64 * TP_SCAN_SPLIT(DK))
    TP_SCAN_SIZES(TP_LAUNCH, d);
#undef TP_LAUNCH
    return tp_check_launch("time_mix_scan");
}

extern "C" long tp_matrix_memory_scan_workspace_floats(int n_seq, int n_chunks, int H, int dk, int dv) {
    return (long)n_seq * n_chunks * H * ((long)dk * dv + dk + 4);
}

// memory [slots, H, dk, dv], normalizer [slots, H, dk], maximum [slots, H], gates [M, 2 H] (input sums, then forget sums), all float32
extern "C" int tp_matrix_memory_scan(const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride, int dtype,
                                     const float* gates, float cap, float q_scale, float* memory, float* normalizer, float* maximum,
                                     const int* slot_ids, const int* cu_rows, float* y, int n_seq, int H, int dk, int dv,
                                     int chunk, int n_chunks, float* workspace, void* stream) {
    TP_REQUIRE(n_seq > 0 && H > 0 && dk > 0 && dv > 0, "matrix_memory_scan: empty shape sequences=%d heads=%d key=%d value=%d", n_seq, H, dk, dv);
    TP_REQUIRE(dk <= 256, "matrix_memory_scan: keys of %d elements exceed the 256 a lane keeps", dk);
    TP_REQUIRE(dv <= 256, "matrix_memory_scan: values of %d elements exceed the 256 columns of a block", dv);
    TP_REQUIRE(H <= 65535, "matrix_memory_scan: %d heads exceed one launch", H);
    TP_REQUIRE(cap > 0.f, "matrix_memory_scan: the gates' cap must be positive");
    TP_REQUIRE(q && k && v && gates && memory && normalizer && maximum && slot_ids && cu_rows && y, "matrix_memory_scan: null operand");
    TP_REQUIRE(chunk == 0 || (chunk > 0 && n_chunks > 0 && workspace && (long)n_seq * n_chunks <= 0x7fffffffL),
               "matrix_memory_scan: %d chunks of %d rows need a workspace", n_chunks, chunk);
    float* ws_aux = workspace ? workspace + (size_t)n_seq * n_chunks * H * ((size_t)dk * dv + dk) : nullptr;
    MatrixMemoryArgs a{q, q_stride, k, k_stride, v, v_stride, gates, cap, q_scale, memory, normalizer, maximum, slot_ids, cu_rows, y, H, dk, dv,
                       chunk, n_chunks, workspace, ws_aux};
    dim3 grid(n_seq, H), chunk_grid(n_seq * (chunk > 0 ? n_chunks : 1), H), carry_grid(n_seq, H, tp_cdiv(dk * dv + dk, 256));
    const int threads = 64 * tp_cdiv(dv, 64);            // times the waves a group of columns is split over
    hipStream_t s = (hipStream_t)stream;
    if (dtype != TP_BF16 && dtype != TP_F32) return tp_fail("matrix_memory_scan: unknown dtype %d", dtype);
#define TP_LAUNCH(DK) TP_SCAN_MODES(matrix_memory_scan_k, (matrix_memory_carry_k<<<carry_grid, 256, 0, s>>>(memory, normalizer, maximum, slot_ids, cu_rows, workspace, ws_aux, H, dk, dv, chunk, n_chunks)), DK, grid, chunk_grid, threads * TP_MM_SPLIT(DK))
    TP_SCAN_SIZES(TP_LAUNCH, dk);
#undef TP_LAUNCH
    return tp_check_launch("matrix_memory_scan");
}
