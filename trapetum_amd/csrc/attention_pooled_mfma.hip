// Matrix-core kernel of the attention over a window plus pooled blocks (see attention_pooled.hip for the mechanism and
// the plain kernel), for bf16 rows of TP_HD elements, TP_HD a multiple of 32 up to 256.  One launch serves prompts,
// portions of prompts and decode steps.
//
// A block of four waves owns 16 consecutive query rows of one sequence, one query head g and one kv head c whose
// values g's weights are applied to.  The keys the 16 queries can see are one list, the pooled blocks 0 .. NB - 1 (NB of
// the tile's last query) and then the positions from the first query's window start to the last query; each query masks
// what it does not see.  The list is cut into chunks of 32 keys that the waves take in turn, every wave with its own
// running maximum, sum and outputs, which meet in LDS once at the end, in wave order.
//
// Scores transposed, S^T = K Q^T, with `v_mfma_f32_16x16x32_bf16`: the A operand is 16 key rows straight from global
// memory (cache pages, pooled pages or the step's rows: a lane computes one key's address and hands it on by lane
// reads), the B operand the queries in registers; a lane gets four keys of one query, so the softmax statistics are
// per-lane scalars and two lane exchanges.  A lane's eight weights of a chunk (two score tiles) are the B operand of the
// second product as they lie, O^T = V^T P^T; the order of the 32 keys in that product's K dimension is then (4j + i of
// the first tile, 4j + i of the second) for lane group j, and V^T is read from an LDS copy of the chunk's value rows
// in that order.  The weights enter the second product as two bf16 terms (a weight's rounding and the rounding's
// remainder), so they meet the values with 16 bits of mantissa.
//
// That kernel (`attn_pooled_tile_k`) is for steps of few rows a sequence (decode steps, short portions): its
// parallelism comes from the keys.  Steps of many rows run `attn_pooled_rows_k`: a block owns 64 consecutive query rows
// of one (g, c), a wave 16 of them, and all four waves walk the same key list (the union of what the 64 queries see),
// whose chunks of 32 key rows and 32 value rows are staged in LDS once for the four of them (two stages taking turns, one
// barrier a chunk; the next chunk's loads travel while the current one is multiplied).  A key row is then read from
// global memory once per 64 queries instead of once per 16, which is what bounds this attention: its keys and values
// come from L2 for every (tile, g, c), far more often than the matrix instructions can be fed otherwise.
#include "common.h"
#include <type_traits>

#ifndef TP_HD
#error "compile with -DTP_HD=<head size>"
#endif

#if TP_HD % 32 == 0

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 pt_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float pt_f32x4;
union PtFrag { uint4 u; pt_bf16x8 v; bf16_t h[8]; };

struct AttnPooledTileArgs {
    const bf16_t* q; long q_stride;
    const bf16_t* k; long k_stride; const bf16_t* v; long v_stride;
    const int* cu_rows; const int* new_len;
    const int* table; int table_w; const bf16_t* k_pool; const bf16_t* v_pool; int page; int rows_cap;
    const int* ptable; int ptable_w; const bf16_t* pk; const bf16_t* pv; int P;
    float* out;
    int H, KV, VG; float scale, cap; int window;
};

namespace {
constexpr int HD = TP_HD, WAVES = 4, CHUNK = 32, KS = HD / 32, VT = HD / 16, VSTRIDE = HD + 8, PIECES = HD / 8;
constexpr int STAGE_BYTES = WAVES * CHUNK * VSTRIDE * 2, MERGE_BYTES = WAVES * HD * 16 * 4;
constexpr int LDS_BYTES = STAGE_BYTES > MERGE_BYTES ? STAGE_BYTES : MERGE_BYTES;

__device__ __forceinline__ const bf16_t* lane_ptr(const bf16_t* p, int lane) {
    const uint64_t x = (uint64_t)p;
    const uint32_t lo = __shfl((int)(uint32_t)x, lane, 64), hi = __shfl((int)(uint32_t)(x >> 32), lane, 64);
    return (const bf16_t*)(((uint64_t)hi << 32) | lo);
}
}

__global__ void __launch_bounds__(256)
attn_pooled_tile_k(AttnPooledTileArgs a) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[LDS_BYTES];
    __shared__ float m_s[WAVES][16], l_s[WAVES][16];
    const int tile = blockIdx.x, seq = blockIdx.y, h = blockIdx.z / a.VG, c = blockIdx.z - h * a.VG;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 15, j = lane >> 4;
    const int first_row = a.cu_rows[seq], count = a.cu_rows[seq + 1] - first_row;
    if (tile * 16 >= count) return;
    const int gk = h / (a.H / a.KV), gv = a.VG > 1 ? c : gk;
    const int start = a.new_len[seq] - count;             // the first position that is a row of the step
    const int r0 = tile * 16, nq = min(16, count - r0);
    const int p0 = start + r0, p_max = p0 + nq - 1;
    const int W = a.window;
    const int LO = W > 0 ? max(0, p0 - W + 1) : 0;
    const int NB = a.P > 0 ? max(0, p_max - W + 1) / a.P : 0;
    const int n_keys = NB + (p_max - LO + 1);
    const int qc = min(col, nq - 1), pq = p0 + qc;         // this lane's query (a column of the score tiles)
    const int my_lo = W > 0 ? max(0, pq - W + 1) : 0, my_nb = a.P > 0 ? max(0, pq - W + 1) / a.P : 0;

    PtFrag qf[KS];
    {
        const bf16_t* qrow = a.q + (size_t)(first_row + r0 + qc) * a.q_stride + (size_t)h * HD + j * 8;
#pragma unroll
        for (int s = 0; s < KS; s++) qf[s].u = *reinterpret_cast<const uint4*>(qrow + s * 32);
    }
    pt_f32x4 acc[VT];
#pragma unroll
    for (int t = 0; t < VT; t++) acc[t] = (pt_f32x4){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    bf16_t* v_lds = reinterpret_cast<bf16_t*>(lds) + (size_t)wave * CHUNK * VSTRIDE;
    // in units of log 2: exponentials are one instruction each, and the cap's tanh is 1 - 2 / (1 + 2^(2 x log2 e))
    constexpr float LOG2E = 1.4426950408889634f;
    const float soc2 = a.cap > 0.f ? 2.f * LOG2E * a.scale / a.cap : 0.f, cap2 = a.cap * LOG2E, scale2 = a.scale * LOG2E;
    const int psh = 31 - __clz(a.page), pmask = a.page - 1;          // the page size is a power of two (checked on the host)
    const float inv_ring = a.rows_cap > 0 ? 1.f / (float)a.rows_cap : 0.f;

    // where a chunk's 32 keys and values lie (lane l works out key l % 32), and the loads of both: the keys' rows into
    // the first product's A operands, the values' rows into registers on their way to LDS
    constexpr int NV = CHUNK * PIECES / 64;
    pt_bf16x8 vr[NV];                                    // (a native vector: an array of uint4 structs stays in scratch memory)
    PtFrag kbuf[2][2][KS];                               // two sets of key operands that take turns
#define PT_FETCH(U0, B) do { \
    const int u0_ = (U0); \
        const bf16_t *kp, *vp; \
        const int u = min(u0_ + (lane & 31), n_keys - 1);   /* past the last key: a row that exists, masked below */ \
        if (u < NB) { \
            const int pg = a.ptable[(size_t)seq * a.ptable_w + (u >> psh)]; \
            const size_t at = (((size_t)pg * a.KV) << psh) + (u & pmask); \
            kp = a.pk + (at + (size_t)gk * a.page) * HD; \
            vp = a.pv + (at + (size_t)gv * a.page) * HD; \
        } else { \
            const int t = LO + u - NB; \
            if (t < start) { \
                int row = t - (int)((float)t * inv_ring) * a.rows_cap;     /* t % rows_cap: positions stay below 2^24 */ \
                row += row < 0 ? a.rows_cap : 0; \
                row -= row >= a.rows_cap && a.rows_cap > 0 ? a.rows_cap : 0; \
                const int pg = a.table[(size_t)seq * a.table_w + (row >> psh)]; \
                const size_t at = (((size_t)pg * a.KV) << psh) + (row & pmask); \
                kp = a.k_pool + (at + (size_t)gk * a.page) * HD; \
                vp = a.v_pool + (at + (size_t)gv * a.page) * HD; \
            } else { \
                const size_t row = (size_t)(first_row + t - start); \
                kp = a.k + row * a.k_stride + (size_t)gk * HD; \
                vp = a.v + row * a.v_stride + (size_t)gv * HD; \
            } \
        } \
_Pragma("unroll") \
        for (int t = 0; t < 2; t++) { \
            const bf16_t* mine = lane_ptr(kp, t * 16 + col) + j * 8; \
_Pragma("unroll") \
            for (int s = 0; s < KS; s++) kbuf[B][t][s].u = *reinterpret_cast<const uint4*>(mine + s * 32); \
        } \
_Pragma("unroll") \
        for (int i = 0; i < NV; i++) { \
            const int idx = lane + 64 * i, key = idx / PIECES, piece = idx - key * PIECES; \
            vr[i] = *reinterpret_cast<const pt_bf16x8*>(lane_ptr(vp, key) + piece * 8); \
        } \
} while (0)
    PT_FETCH(wave * CHUNK, 0);                          // (a wave without a chunk reads rows that exist and uses none)
    // two chunks a round, the key operands' two register sets taking turns
    for (int u2 = wave * CHUNK; u2 < n_keys; u2 += 2 * WAVES * CHUNK) {
#pragma unroll
    for (int B = 0; B < 2; B++) {
        const int u0 = u2 + B * WAVES * CHUNK;
        if (u0 >= n_keys) break;
        // the chunk's value rows into this wave's part of LDS; then the next chunk's loads are asked for, so that they
        // travel while this chunk is worked on (always, from clamped addresses: a load behind a branch is waited for)
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int idx = lane + 64 * i, key = idx / PIECES, piece = idx - key * PIECES;
            *reinterpret_cast<pt_bf16x8*>(v_lds + key * VSTRIDE + piece * 8) = vr[i];
        }
        PT_FETCH(u0 + WAVES * CHUNK, 1 - B);
        // ---- scores: two tiles of 16 keys; lane (col, j) gets keys 4j .. 4j + 3 of each for query col ------------------
        pt_f32x4 sc[2];
        float pr[2][4];
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; t++) {
            sc[t] = (pt_f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; s++) sc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kbuf[B][t][s].v, qf[s].v, sc[t], 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int u = u0 + t * 16 + j * 4 + i, pos = LO + u - NB;
                const bool seen = u < n_keys && (u < NB ? u < my_nb : (pos >= my_lo && pos <= pq));
                const float x = a.cap > 0.f ? cap2 - 2.f * cap2 * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(sc[t][i] * soc2))
                                            : sc[t][i] * scale2;
                pr[t][i] = seen ? x : -INFINITY;
                mx = fmaxf(mx, pr[t][i]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        float alpha = 1.f, psum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                pr[t][i] = m_new == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(pr[t][i] - m_new);
                psum += pr[t][i];
            }
        if (m_new != -INFINITY) alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        psum += __shfl_xor(psum, 16, 64);
        psum += __shfl_xor(psum, 32, 64);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        PtFrag ph, pl;                                   // the weights as two bf16 terms
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const __bf16 hi = (__bf16)pr[t][i];
                ph.v[t * 4 + i] = hi;
                pl.v[t * 4 + i] = (__bf16)(pr[t][i] - (float)hi);
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // ---- O^T += V^T P^T.  Row r of output tile vt is head element r VT + vt, so that a lane (r = col) finds the
        // elements of all its tiles side by side in a value row: it reads VT elements of each of its eight keys (4j + i of
        // both tiles) in wide LDS reads and puts the operands together in registers
        uint32_t vw[8][VT / 2];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const uint32_t* src = reinterpret_cast<const uint32_t*>(v_lds + ((e < 4 ? 0 : 12) + 4 * j + e) * VSTRIDE + col * VT);
#pragma unroll
            for (int x = 0; x < VT / 2; x++) vw[e][x] = src[x];
        }
        PtFrag vfs[VT];
#pragma unroll
        for (int vt = 0; vt < VT; vt++) {
            PtFrag vf;
#pragma unroll
            for (int e = 0; e < 8; e++) vf.h[e] = (bf16_t)(vw[e][vt >> 1] >> (16 * (vt & 1)));
            vfs[vt] = vf;
            acc[vt] *= alpha;
            acc[vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, ph.v, acc[vt], 0, 0, 0);
        }
#pragma unroll
        for (int vt = 0; vt < VT; vt++)                   // the second terms afterwards: no instruction waits for the one before it
            acc[vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vfs[vt].v, pl.v, acc[vt], 0, 0, 0);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    }
#undef PT_FETCH
    // ---- the waves' parts meet, in wave order ------------------------------------------------------------------------------
    __syncthreads();                                     // every wave is done with its part of LDS
    float* o_s = reinterpret_cast<float*>(lds);          // [wave][VT][4][64]
    if (j == 0) { m_s[wave][col] = m_run; l_s[wave][col] = l_run; }
#pragma unroll
    for (int vt = 0; vt < VT; vt++)
#pragma unroll
        for (int i = 0; i < 4; i++) o_s[((size_t)(wave * VT + vt) * 4 + i) * 64 + lane] = acc[vt][i];
    __syncthreads();
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; w++) M = fmaxf(M, m_s[w][col]);
    float f[WAVES], L = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; w++) {
        f[w] = m_s[w][col] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_s[w][col] - M);
        L += l_s[w][col] * f[w];
    }
    const float inv = 1.f / L;
    if (col < nq) {
        float* orow = a.out + (((size_t)(first_row + r0 + col) * a.H + h) * a.VG + c) * HD;
        for (int vt = wave; vt < VT; vt += WAVES) {
            float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
            float* oe = reinterpret_cast<float*>(&o);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; w++) s += o_s[((size_t)(w * VT + vt) * 4 + i) * 64 + lane] * f[w];
                oe[i] = s * inv;
            }
#pragma unroll
            for (int i = 0; i < 4; i++) orow[(j * 4 + i) * VT + vt] = oe[i];
        }
    }
}


// ---- steps of many rows: 64 query rows a block, key and value chunks shared through LDS -------------------------------------
namespace {
constexpr int KSTRIDE = HD + 8, ROWS_STAGE = CHUNK * (KSTRIDE + VSTRIDE) * 2;      // bytes of one stage: 32 key rows, 32 value rows
constexpr int NLOAD = (CHUNK * PIECES + 255) / 256;                                // 16-byte pieces a thread moves per chunk and kind
}

__global__ void __launch_bounds__(256, 2)
attn_pooled_rows_k(AttnPooledTileArgs a) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * ROWS_STAGE];
    const int seq = blockIdx.y, h = blockIdx.z / a.VG, c = blockIdx.z - h * a.VG;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 15, j = lane >> 4;
    const int first_row = a.cu_rows[seq], count = a.cu_rows[seq + 1] - first_row;
    if (blockIdx.x * 64 >= count) return;
    const int gk = h / (a.H / a.KV), gv = a.VG > 1 ? c : gk;
    const int start = a.new_len[seq] - count;
    const int W = a.window;
    // the block's rows and the one key list of all of them
    const int b0 = blockIdx.x * 64, bn = min(64, count - b0);
    const int bp0 = start + b0, bp_max = bp0 + bn - 1;
    const int LO = W > 0 ? max(0, bp0 - W + 1) : 0;
    const int NB = a.P > 0 ? max(0, bp_max - W + 1) / a.P : 0;
    const int n_keys = NB + (bp_max - LO + 1);
    // this wave's 16 rows (a wave past the step's rows helps with the loads and computes nothing)
    const int r0 = b0 + wave * 16, nq = min(16, count - r0);
    const bool active = nq > 0;
    const int p0 = start + r0, p_max = p0 + max(nq, 1) - 1;
    const int qc = min(col, max(nq, 1) - 1), pq = p0 + qc;
    const int my_lo = W > 0 ? max(0, pq - W + 1) : 0, my_nb = a.P > 0 ? max(0, pq - W + 1) / a.P : 0;
    const int w_lo = W > 0 ? max(0, p0 - W + 1) : 0, w_nb = a.P > 0 ? max(0, p_max - W + 1) / a.P : 0;     // of the wave's rows together

    PtFrag qf[KS];
    {
        const bf16_t* qrow = a.q + (size_t)(first_row + min(r0 + qc, count - 1)) * a.q_stride + (size_t)h * HD + j * 8;
#pragma unroll
        for (int s = 0; s < KS; s++) qf[s].u = *reinterpret_cast<const uint4*>(qrow + s * 32);
    }
    pt_f32x4 acc[VT];
#pragma unroll
    for (int t = 0; t < VT; t++) acc[t] = (pt_f32x4){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    constexpr float LOG2E = 1.4426950408889634f;
    const float soc2 = a.cap > 0.f ? 2.f * LOG2E * a.scale / a.cap : 0.f, cap2 = a.cap * LOG2E, scale2 = a.scale * LOG2E;
    const int psh = 31 - __clz(a.page), pmask = a.page - 1;
    const float inv_ring = a.rows_cap > 0 ? 1.f / (float)a.rows_cap : 0.f;

    pt_bf16x8 kr[NLOAD], vr[NLOAD];
    // a chunk's rows on their way to LDS: lane l works out where key l % 32 and its value lie; thread x moves the pieces
    // x, x + 256, ... of the chunk's 32 x PIECES, of keys and of values
#define PT_LOAD(U0) do { \
        const bf16_t *kp, *vp; \
        const int u = min((U0) + (lane & 31), n_keys - 1); \
        if (u < NB) { \
            const int pg = a.ptable[(size_t)seq * a.ptable_w + (u >> psh)]; \
            const size_t at = (((size_t)pg * a.KV) << psh) + (u & pmask); \
            kp = a.pk + (at + ((size_t)gk << psh)) * HD; \
            vp = a.pv + (at + ((size_t)gv << psh)) * HD; \
        } else { \
            const int t = LO + u - NB; \
            if (t < start) { \
                int row = t - (int)((float)t * inv_ring) * a.rows_cap; \
                row += row < 0 ? a.rows_cap : 0; \
                row -= row >= a.rows_cap && a.rows_cap > 0 ? a.rows_cap : 0; \
                const int pg = a.table[(size_t)seq * a.table_w + (row >> psh)]; \
                const size_t at = (((size_t)pg * a.KV) << psh) + (row & pmask); \
                kp = a.k_pool + (at + ((size_t)gk << psh)) * HD; \
                vp = a.v_pool + (at + ((size_t)gv << psh)) * HD; \
            } else { \
                const size_t row = (size_t)(first_row + t - start); \
                kp = a.k + row * a.k_stride + (size_t)gk * HD; \
                vp = a.v + row * a.v_stride + (size_t)gv * HD; \
            } \
        } \
_Pragma("unroll") \
        for (int i = 0; i < NLOAD; i++) { \
            const int idx = threadIdx.x + 256 * i, key = min(idx / PIECES, CHUNK - 1), piece = idx % PIECES; \
            kr[i] = *reinterpret_cast<const pt_bf16x8*>(lane_ptr(kp, key) + piece * 8); \
            vr[i] = *reinterpret_cast<const pt_bf16x8*>(lane_ptr(vp, key) + piece * 8); \
        } \
    } while (0)
    PT_LOAD(0);
    int stage = 0;
    for (int u0 = 0; u0 < n_keys; u0 += CHUNK, stage ^= 1) {
        bf16_t* k_lds = reinterpret_cast<bf16_t*>(lds + stage * ROWS_STAGE);
        bf16_t* v_lds = k_lds + CHUNK * KSTRIDE;
#pragma unroll
        for (int i = 0; i < NLOAD; i++) {
            const int idx = threadIdx.x + 256 * i, key = idx / PIECES, piece = idx % PIECES;
            if (key < CHUNK) {
                *reinterpret_cast<pt_bf16x8*>(k_lds + key * KSTRIDE + piece * 8) = kr[i];
                *reinterpret_cast<pt_bf16x8*>(v_lds + key * VSTRIDE + piece * 8) = vr[i];
            }
        }
        PT_LOAD(u0 + CHUNK);                              // the next chunk travels while this one is worked on
        __syncthreads();                                   // the stage is whole; the other stage is free once every wave is here
        // a chunk none of the wave's 16 rows can see (positions after its last row or before its first row's window,
        // blocks that are not whole before it) costs it nothing
        const bool blocks_seen = u0 < w_nb, tokens_seen = u0 + CHUNK > NB && LO + (u0 + CHUNK - 1) - NB >= w_lo && LO + max(u0, NB) - NB <= p_max;
        if (!active || !(blocks_seen || tokens_seen)) continue;
        pt_f32x4 sc[2];
        float pr[2][4];
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; t++) {
            sc[t] = (pt_f32x4){0.f, 0.f, 0.f, 0.f};
            const bf16_t* krow = k_lds + (t * 16 + col) * KSTRIDE + j * 8;
            pt_f32x4 odd = (pt_f32x4){0.f, 0.f, 0.f, 0.f};     // two chains of sums a tile: an instruction waits for every second one before it only
#pragma unroll
            for (int s = 0; s < KS; s++) {
                PtFrag kf;
                kf.v = *reinterpret_cast<const pt_bf16x8*>(krow + s * 32);
                if (s & 1) odd = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qf[s].v, odd, 0, 0, 0);
                else sc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qf[s].v, sc[t], 0, 0, 0);
            }
            sc[t] += odd;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int u = u0 + t * 16 + j * 4 + i, pos = LO + u - NB;
                const bool seen = u < n_keys && (u < NB ? u < my_nb : (pos >= my_lo && pos <= pq));
                const float x = a.cap > 0.f ? cap2 - 2.f * cap2 * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(sc[t][i] * soc2))
                                            : sc[t][i] * scale2;
                pr[t][i] = seen ? x : -INFINITY;
                mx = fmaxf(mx, pr[t][i]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        float alpha = 1.f, psum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                pr[t][i] = m_new == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(pr[t][i] - m_new);
                psum += pr[t][i];
            }
        if (m_new != -INFINITY) alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        psum += __shfl_xor(psum, 16, 64);
        psum += __shfl_xor(psum, 32, 64);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        PtFrag ph, pl;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const __bf16 hi = (__bf16)pr[t][i];
                ph.v[t * 4 + i] = hi;
                pl.v[t * 4 + i] = (__bf16)(pr[t][i] - (float)hi);
            }
        // the value rows' elements in two halves of the output tiles, so that a wave keeps to 256 registers and two
        // blocks share a CU
        constexpr int HALVES = VT % 4 == 0 ? 2 : 1, VH = VT / HALVES;       // (a half holds whole pairs of tiles)
#pragma unroll
        for (int hf = 0; hf < HALVES; hf++) {
            uint32_t vw[8][VH / 2];
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const uint32_t* src = reinterpret_cast<const uint32_t*>(v_lds + ((e < 4 ? 0 : 12) + 4 * j + e) * VSTRIDE + col * VT + hf * VH);
#pragma unroll
                for (int x = 0; x < VH / 2; x++) vw[e][x] = src[x];
            }
            PtFrag vfs[VH];
#pragma unroll
            for (int v2 = 0; v2 < VH; v2++) {
                const int vt = hf * VH + v2;
                PtFrag vf;
#pragma unroll
                for (int e = 0; e < 8; e++) vf.h[e] = (bf16_t)(vw[e][v2 >> 1] >> (16 * (v2 & 1)));
                vfs[v2] = vf;
                acc[vt] *= alpha;
                acc[vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, ph.v, acc[vt], 0, 0, 0);
            }
#pragma unroll
            for (int v2 = 0; v2 < VH; v2++)               // the second terms afterwards: no instruction waits for the one before it
                acc[hf * VH + v2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vfs[v2].v, pl.v, acc[hf * VH + v2], 0, 0, 0);
        }
    }
#undef PT_LOAD
    if (active && col < nq) {
        const float inv = 1.f / l_run;
        float* orow = a.out + (((size_t)(first_row + r0 + col) * a.H + h) * a.VG + c) * HD;
#pragma unroll
        for (int vt = 0; vt < VT; vt++)
#pragma unroll
            for (int i = 0; i < 4; i++) orow[(j * 4 + i) * VT + vt] = acc[vt][i] * inv;
    }
}

extern "C" int tp_attn_pooled_tile(const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride,
                                   int n_seq, int max_count, int H, int KV, const int* cu_rows, const int* new_len,
                                   const int* table, int table_w, const void* k_pool, const void* v_pool, int page, int rows_cap,
                                   const int* ptable, int ptable_w, const void* pk, const void* pv, int P,
                                   float scale, float cap, int window, int all_values, float* out, void* stream) {
    TP_REQUIRE(n_seq > 0 && max_count > 0 && H > 0 && KV > 0 && H % KV == 0, "attention (pooled): shape sequences=%d rows=%d heads=%d kv=%d", n_seq, max_count, H, KV);
    TP_REQUIRE(q && k && v && cu_rows && new_len && out && table && k_pool && v_pool && page > 0 && table_w > 0, "attention (pooled): null operand");
    TP_REQUIRE(rows_cap >= 0 && (rows_cap == 0 || rows_cap % page == 0), "attention (pooled): ring of %d rows is no multiple of the page size %d", rows_cap, page);
    TP_REQUIRE((page & (page - 1)) == 0, "attention (pooled, matrix cores): the page size %d is no power of two", page);
    TP_REQUIRE(P >= 0 && (P == 0 || (window > 0 && ptable && pk && pv && ptable_w > 0)), "attention (pooled): blocks of %d positions need a window, their page table and pools", P);
    TP_REQUIRE(q_stride % 8 == 0 && k_stride % 8 == 0 && v_stride % 8 == 0, "attention (pooled): row strides must be whole 16-byte pieces");
    for (const void* p : {q, k, v, k_pool, v_pool, pk, pv, (const void*)out})
        TP_REQUIRE((uintptr_t)p % 16 == 0, "attention (pooled): operands must be aligned to 16 bytes");
    const int VG = all_values ? KV : 1;
    TP_REQUIRE(n_seq <= 65535 && (long)H * VG <= 65535, "attention (pooled): %d sequences or %d head pairs exceed one launch", n_seq, H * VG);
    AttnPooledTileArgs a{};
    a.q = (const bf16_t*)q; a.q_stride = q_stride; a.k = (const bf16_t*)k; a.k_stride = k_stride; a.v = (const bf16_t*)v; a.v_stride = v_stride;
    a.cu_rows = cu_rows; a.new_len = new_len; a.table = table; a.table_w = table_w; a.k_pool = (const bf16_t*)k_pool; a.v_pool = (const bf16_t*)v_pool;
    a.page = page; a.rows_cap = rows_cap; a.ptable = ptable; a.ptable_w = ptable_w; a.pk = (const bf16_t*)pk; a.pv = (const bf16_t*)pv; a.P = P;
    a.out = out; a.H = H; a.KV = KV; a.VG = VG; a.scale = scale; a.cap = cap; a.window = window;
    if (max_count > 32) {                                 // many rows a sequence: 64 a block, the keys' chunks shared
        dim3 grid(tp_cdiv(max_count, 64), n_seq, H * VG);
        attn_pooled_rows_k<<<grid, 256, 0, (hipStream_t)stream>>>(a);
    } else {
        dim3 grid(tp_cdiv(max_count, 16), n_seq, H * VG);
        attn_pooled_tile_k<<<grid, 256, 0, (hipStream_t)stream>>>(a);
    }
    return tp_check_launch("attention (pooled, matrix cores)");
}

#else

extern "C" int tp_attn_pooled_tile(const void*, long, const void*, long, const void*, long, int, int, int, int, const int*, const int*,
                                   const int*, int, const void*, const void*, int, int, const int*, int, const void*, const void*, int,
                                   float, float, int, int, float*, void*) {
    return tp_fail("attention (pooled, matrix cores): head size %d is no multiple of 32", TP_HD);
}

#endif
