// Attention through a cached latent: what stands between the input projection and the attention kernels, and the
// per-head products that carry queries into the latent's space and weighted latents out of it.
#include "common.h"
#include "tile.h"
#include "tile_mfma.h"

// ---- a step's projections -> rotated query parts, and the rows [rope(key part) | rmsnorm(latent) * gain] ----------
// proj row: H heads of [dr rotated | dn unrotated] query elements, then (own) [dr key part | R latent].
// q row: H heads of [dr | R]; this kernel fills the first dr of each (the rest is a product's output).
// The first `rot` of the dr elements turn in pairs (f, f + rot / 2) by pos * inv_freq[f]; the others pass.
// grid (rows); dynamic LDS: rot floats (cosines, sines).
template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_k(const T* __restrict__ proj, long proj_stride, int H, int dn, int dr, int R,
                 const float* __restrict__ gain, float eps, const float* __restrict__ inv_freq, int rot,
                 const int* __restrict__ row_seq, const int* __restrict__ row_pos, const int* __restrict__ new_len,
                 const int* __restrict__ table, int table_w, T* __restrict__ pool, int page, int rows_cap,
                 T* __restrict__ q, T* __restrict__ mine, int own, const T* __restrict__ tail_rows, long tail_stride) {
    extern __shared__ float cs[];                        // [rot / 2] cosines, [rot / 2] sines
    __shared__ float red[16];
    const int r = blockIdx.x, pos = row_pos[r], half = rot / 2, row = dr + R;
    for (int f = threadIdx.x; f < half; f += blockDim.x) {
        const float ang = (float)pos * inv_freq[f];
        cs[f] = cosf(ang);
        cs[half + f] = sinf(ang);
    }
    __syncthreads();
    const T* pr = proj + (size_t)r * proj_stride;
    T* qr = q + (size_t)r * H * row;
    for (int item = threadIdx.x; item < H * dr; item += blockDim.x) {
        const int h = item / dr, e = item - h * dr;
        const T* src = pr + (size_t)h * (dr + dn);
        float y;
        if (e < half) y = ld_f32(src + e) * cs[e] - ld_f32(src + e + half) * cs[half + e];
        else if (e < rot) y = ld_f32(src + e) * cs[e - half] + ld_f32(src + e - half) * cs[e];
        else y = ld_f32(src + e);
        st_f32(qr + (size_t)h * row + e, y);
    }
    if (!own) return;
    const T* tail = tail_rows ? tail_rows + (size_t)r * tail_stride : pr + (size_t)H * (dr + dn);     // a product of its own, or the row's end
    T* dst = nullptr;                                    // the row's place in the cache
    if (table) {
        const int seq = row_seq[r];
        int at = pos;
        bool keep = true;
        if (rows_cap > 0) {
            keep = pos + rows_cap >= new_len[seq];       // else a later row of this step takes the same ring row
            at = pos % rows_cap;
        }
        const int pg = keep && at / page < table_w ? table[(size_t)seq * table_w + at / page] : -1;     // a table too narrow for the position caches nothing
        if (pg >= 0) dst = pool + ((size_t)pg * page + at % page) * row;
    }
    T* mr = mine + (size_t)r * row;
    for (int e = threadIdx.x; e < dr; e += blockDim.x) {
        float y;
        if (e < half) y = ld_f32(tail + e) * cs[e] - ld_f32(tail + e + half) * cs[half + e];
        else if (e < rot) y = ld_f32(tail + e) * cs[e - half] + ld_f32(tail + e - half) * cs[e];
        else y = ld_f32(tail + e);
        st_f32(mr + e, y);
        if (dst) st_f32(dst + e, y);
    }
    float ss = 0.f;
    for (int e = threadIdx.x; e < R; e += blockDim.x) { const float v = ld_f32(tail + dr + e); ss += v * v; }
    ss = block_sum(ss, red);
    const float scale = rsqrtf(ss / (float)R + eps);
    for (int e = threadIdx.x; e < R; e += blockDim.x) {
        const float y = (ld_f32(tail + dr + e) * scale) * gain[e];
        st_f32(mr + dr + e, y);
        if (dst) st_f32(dst + dr + e, y);
    }
}

extern "C" int tp_latent_prepare(const void* proj, long proj_stride, int dtype, int M, int H, int dn, int dr, int R,
                                 const float* gain, float eps, const float* inv_freq, int rot,
                                 const int* row_seq, const int* row_pos, const int* new_len,
                                 const int* table, int table_w, void* pool, int page, int rows_cap,
                                 void* q, void* mine, int own, const void* tail, long tail_stride, void* stream) {
    TP_REQUIRE(M > 0 && H > 0 && dn >= 0 && dr >= 0 && R > 0, "latent_prepare: empty shape M=%d H=%d dn=%d dr=%d R=%d", M, H, dn, dr, R);
    TP_REQUIRE(proj && q && row_pos, "latent_prepare: a null operand");
    TP_REQUIRE(rot >= 0 && rot <= dr && rot % 2 == 0, "latent_prepare: %d turning elements must be even and at most the rotated part's %d", rot, dr);
    TP_REQUIRE(rot == 0 || inv_freq, "latent_prepare: a rotation needs its frequency table");
    TP_REQUIRE(proj_stride >= (long)H * (dr + dn) + (own && !tail ? dr + R : 0), "latent_prepare: rows of %ld elements are too short", proj_stride);
    TP_REQUIRE(!tail || (own && tail_stride >= dr + R), "latent_prepare: the key part and latent as rows of their own need %d elements a row", dr + R);
    TP_REQUIRE(!own || (mine && gain && row_seq && new_len), "latent_prepare: a layer with a latent of its own needs its gain and the rows' output");
    TP_REQUIRE(!table || (pool && page > 0 && table_w > 0), "latent_prepare: a page table without a cache pool");
    if (!table) { page = 1; rows_cap = 0; }
    TP_REQUIRE(rows_cap >= 0 && (rows_cap == 0 || rows_cap % page == 0), "latent_prepare: ring of %d rows is no multiple of the page size %d", rows_cap, page);
    TP_REQUIRE(rot * sizeof(float) <= 32768, "latent_prepare: %d turning elements exceed the kernel's table", rot);
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)rot * sizeof(float);
    if (dtype == TP_BF16)
        latent_prepare_k<bf16_t><<<M, 256, lds, s>>>((const bf16_t*)proj, proj_stride, H, dn, dr, R, gain, eps, inv_freq, rot, row_seq, row_pos,
            new_len, table, table_w, (bf16_t*)pool, page, rows_cap, (bf16_t*)q, (bf16_t*)mine, own, (const bf16_t*)tail, tail_stride);
    else if (dtype == TP_F32)
        latent_prepare_k<float><<<M, 256, lds, s>>>((const float*)proj, proj_stride, H, dn, dr, R, gain, eps, inv_freq, rot, row_seq, row_pos,
            new_len, table, table_w, (float*)pool, page, rows_cap, (float*)q, (float*)mine, own, (const float*)tail, tail_stride);
    else return tp_fail("latent_prepare: unknown dtype %d", dtype);
    return tp_check_launch("latent_prepare");
}

// ---- per-head products: out[m, h, n] = sum_k x[m, h, k] * w[h, n, k] ----------------------------------------------
// x and out are views of wider rows (strides in elements: row, head; elements of a head contiguous); w is contiguous.
// grid (column tiles, row tiles, heads)
template <typename T, int TM>
__global__ void __launch_bounds__(256)
head_linear_k(const T* __restrict__ x, long x_row, long x_head, const T* __restrict__ w, T* __restrict__ out, long o_row, long o_head,
              int M, int N, int K) {
    constexpr int TN = 64, BK = 16;
    __shared__ TileShared<TM, TN, BK> sh;
    const int h = blockIdx.z, m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
    const T* xh = x + (size_t)h * x_head;
    const T* wh = w + (size_t)h * N * K;
    float acc[TM / 16][TN / 16];
    tile_product<TM, TN, BK>(acc, K,
        [&](int m, int k) { return m0 + m < M ? ld_f32(xh + (size_t)(m0 + m) * x_row + k) : 0.f; },
        [&](int n, int k) { return n0 + n < N ? ld_f32(wh + (size_t)(n0 + n) * K + k) : 0.f; }, sh);
    const int ty = threadIdx.x >> 4, tx = threadIdx.x & 15;
#pragma unroll
    for (int i = 0; i < TM / 16; i++)
#pragma unroll
        for (int j = 0; j < TN / 16; j++) {
            const int m = m0 + ty + 16 * i, n = n0 + tx + 16 * j;
            if (m < M && n < N) st_f32(out + (size_t)m * o_row + (size_t)h * o_head + n, acc[i][j]);
        }
}

// the same on the matrix cores: bf16, K a multiple of 8, every head's rows starting on 16 bytes
template <int TM>
__global__ void __launch_bounds__(256)
head_linear_mfma_k(const bf16_t* __restrict__ x, long x_row, long x_head, const bf16_t* __restrict__ w, bf16_t* __restrict__ out,
                   long o_row, long o_head, int M, int N, int K) {
    using Tile = MfmaTile<TM, false>;
    __shared__ typename Tile::Shared sh;
    const int h = blockIdx.z, m0 = blockIdx.y * TM, n0 = blockIdx.x * 64;
    const bf16_t* xh = x + (size_t)h * x_head;
    const bf16_t* wh = w + (size_t)h * N * K;
    const uint4 zero = make_uint4(0, 0, 0, 0);
    const bool wide = o_row % 4 == 0 && o_head % 4 == 0 && (uintptr_t)out % 8 == 0;
    Tile t;
    t.run(K,
        [&](int m, int k) { return m0 + m < M ? *reinterpret_cast<const uint4*>(xh + (size_t)(m0 + m) * x_row + k) : zero; },
        [&](int n, int k) { return n0 + n < N ? *reinterpret_cast<const uint4*>(wh + (size_t)(n0 + n) * K + k) : zero; }, sh);
#pragma unroll
    for (int i = 0; i < Tile::MI; i++)
#pragma unroll
        for (int j = 0; j < Tile::NJ; j++) {
            const int m = m0 + Tile::m_of(i), n = n0 + Tile::n_of(j);
            if (m >= M) continue;
            bf16_t* dst = out + (size_t)m * o_row + (size_t)h * o_head + n;
            if (wide && n + 3 < N) {                      // the lane's four neighbours in one store
                uint2 o;
                o.x = (uint32_t)f32_to_bf16(t.acc[0][i][j][0]) | ((uint32_t)f32_to_bf16(t.acc[0][i][j][1]) << 16);
                o.y = (uint32_t)f32_to_bf16(t.acc[0][i][j][2]) | ((uint32_t)f32_to_bf16(t.acc[0][i][j][3]) << 16);
                *reinterpret_cast<uint2*>(dst) = o;
                continue;
            }
#pragma unroll
            for (int v = 0; v < 4; v++)
                if (n + v < N) dst[v] = f32_to_bf16(t.acc[0][i][j][v]);
        }
}

extern "C" int tp_head_linear(const void* x, long x_row, long x_head, const void* w, void* out, long o_row, long o_head,
                              int dtype, int M, int H, int N, int K, int plain, void* stream) {
    TP_REQUIRE(M > 0 && H > 0 && N > 0 && K > 0, "head_linear: empty shape M=%d H=%d N=%d K=%d", M, H, N, K);
    TP_REQUIRE(x && w && out, "head_linear: a null operand");
    TP_REQUIRE(x_head >= K && o_head >= N && x_row >= (long)(H - 1) * x_head + K && o_row >= (long)(H - 1) * o_head + N,
               "head_linear: strides (%ld, %ld) -> (%ld, %ld) do not hold %d heads of %d -> %d elements", x_row, x_head, o_row, o_head, H, K, N);
    TP_REQUIRE(H <= 65535, "head_linear: %d heads exceed one launch", H);
    hipStream_t s = (hipStream_t)stream;
    const bool few = M <= 16;
    const int TM = few ? 16 : 64;
    dim3 grid(tp_cdiv(N, 64), tp_cdiv(M, TM), H);
    TP_REQUIRE(grid.y <= 65535, "head_linear: %d rows exceed one launch", M);
    if (dtype == TP_BF16 && !plain && M >= 512 && K % 8 == 0 && x_row % 8 == 0 && x_head % 8 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0) {
        grid.y = tp_cdiv(M, 128);
        head_linear_mfma_k<128><<<grid, 256, 0, s>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w, (bf16_t*)out, o_row, o_head, M, N, K);
        return tp_check_launch("head_linear (matrix cores)");
    }
    if (dtype == TP_BF16 && !plain && K % 8 == 0 && x_row % 8 == 0 && x_head % 8 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0) {
        if (few) head_linear_mfma_k<16><<<grid, 256, 0, s>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w, (bf16_t*)out, o_row, o_head, M, N, K);
        else head_linear_mfma_k<64><<<grid, 256, 0, s>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w, (bf16_t*)out, o_row, o_head, M, N, K);
        return tp_check_launch("head_linear (matrix cores)");
    }
#define TP_HEAD_LINEAR(T, TMv) head_linear_k<T, TMv><<<grid, 256, 0, s>>>((const T*)x, x_row, x_head, (const T*)w, (T*)out, o_row, o_head, M, N, K)
    if (dtype == TP_BF16) { if (few) TP_HEAD_LINEAR(bf16_t, 16); else TP_HEAD_LINEAR(bf16_t, 64); }
    else if (dtype == TP_F32) { if (few) TP_HEAD_LINEAR(float, 16); else TP_HEAD_LINEAR(float, 64); }
    else return tp_fail("head_linear: unknown dtype %d", dtype);
#undef TP_HEAD_LINEAR
    return tp_check_launch("head_linear");
}
