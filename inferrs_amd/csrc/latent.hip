// Latent attention: keys and values of all heads are products of ONE low-rank row a token, so only that row (and a
// rotated key part that the heads share) is cached, and the heads' own matrices move to the query side and behind
// the attention:
//     score_h = (W_uk,h^T q_h) . c + q_rot,h . k_rot        out_h = W_uv,h (sum_j p_j c_j)
// The cache row of a token is [c | k_rot]; with the query [W_uk,h^T q_h | q_rot,h] the attention is the ordinary
// one with a single key/value head whose values are the key rows themselves.
//
// Here: (1) what stands between the projections and the attention (norm of the latent row in 32-bit, rotation of
// the shared key part and of the queries' rotated parts, the cache writes), (2) a product with a matrix of its own
// for every head (also used for block-diagonal matrices: a block is a head).
#include "api.h"
#include "common.h"
#include "tile_fma.h"
#include "tile_mfma.h"

// proj[t] = [.. q (H x (d + r)) at q_off .. | down (rank + r) at down_off ..]; q_out [n, H, rank + r] gets the
// rotated parts at [rank, rank + r).  Of a rotated part the first `rd` features turn (i paired with i + rd / 2), the
// rest pass (`interleaved`: 2 i paired with 2 i + 1 instead).  cos / sin [n, rd / 2] are multiplied by `mag`.  The key row goes to k_cache [pages][page][D] and, once
// more, transposed to v_cache [pages][D][page] (D = rank + r), at slot slots[t]; slots null: no cache write.
template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, const T* __restrict__ proj,
    const float* __restrict__ norm_w, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ slots, int H, int d, int r, int rank, int rd, int q_off, int down_off, int ld_proj,
    int page_size, float eps, float mag, int interleaved, const T* __restrict__ qrows, int ld_q) {
    // qrows: null, or the queries' rows where they are no part of `proj` (a product of their own): [n, ld_q], q at q_off
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const int D = rank + r, half = rd / 2;
    const T* row = proj + (long long)t * ld_proj;
    const T* down = row + down_off;
    float sq = 0.f;
    for (int j = threadIdx.x; j < rank; j += blockDim.x) {
        const float v = ld(down + j);
        sq = fmaf(v, v, sq);
    }
    const float rs = 1.0f / sqrtf(block_sum(sq, scratch) / (float)rank + eps);
    const float* cs = cos_t != nullptr ? cos_t + (long long)t * half : nullptr;
    const float* sn = sin_t != nullptr ? sin_t + (long long)t * half : nullptr;
    if (slots != nullptr) {
        const int slot = slots[t];
        const int page = slot / page_size, off = slot - page * page_size;
        T* krow = k_cache + ((long long)page * page_size + off) * D;
        T* vcol = v_cache + (long long)page * D * page_size + off;
        for (int j = threadIdx.x; j < D; j += blockDim.x) {
            float v;
            if (j < rank) {
                v = ld(down + j) * rs * norm_w[j];
            } else {
                const int i = j - rank;
                const T* kr = down + rank;
                if (cs != nullptr && i < rd) {
                    // (pair p: features p and p + rd / 2, or, interleaved, 2 p and 2 p + 1; `first`: this is the pair's first)
                    const bool first = interleaved ? (i & 1) == 0 : i < half;
                    const int p = interleaved ? i >> 1 : (i < half ? i : i - half);
                    const int ia = interleaved ? 2 * p : p, ib = interleaved ? 2 * p + 1 : p + half;
                    const float a = ld(kr + ia), b = ld(kr + ib), c = cs[p] * mag, s = sn[p] * mag;
                    v = first ? a * c - b * s : b * c + a * s;
                } else {
                    v = ld(kr + i);
                }
            }
            st(krow + j, v);
            st(vcol + (long long)j * page_size, v);
        }
    }
    for (int idx = threadIdx.x; idx < H * r; idx += blockDim.x) {
        const int hh = idx / r, i = idx - hh * r;
        const T* qr = (qrows != nullptr ? qrows + (long long)t * ld_q : row) + q_off + (long long)hh * (d + r) + d;
        float v;
        if (cs != nullptr && i < rd) {
            const bool first = interleaved ? (i & 1) == 0 : i < half;
            const int p = interleaved ? i >> 1 : (i < half ? i : i - half);
            const int ia = interleaved ? 2 * p : p, ib = interleaved ? 2 * p + 1 : p + half;
            const float a = ld(qr + ia), b = ld(qr + ib), c = cs[p] * mag, s = sn[p] * mag;
            v = first ? a * c - b * s : b * c + a * s;
        } else {
            v = ld(qr + i);
        }
        st(q_out + ((long long)t * H + hh) * D + rank + i, v);
    }
}

extern "C" int ia_latent_prep(void* q_out, void* k_cache, void* v_cache, const void* proj, const float* norm_w,
                              const float* cos_t, const float* sin_t, const int* slots, int n, int H, int d, int r,
                              int rank, int rd, int q_off, int down_off, int ld_proj, int page_size, float eps,
                              float mag, int interleaved, const void* qrows, int ld_q, int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && H > 0 && d > 0 && r >= 0 && rank > 0 && rd >= 0 && rd <= r && rd % 2 == 0 && page_size > 0,
             "latent_prep: bad sizes n=%d heads=%d dim=%d rot_dim=%d rank=%d rotated=%d page=%d", n, H, d, r, rank, rd,
             page_size);
    IA_CHECK(q_off >= 0 && down_off >= 0 && q_off + H * (d + r) <= (qrows != nullptr ? ld_q : ld_proj) && down_off + rank + r <= ld_proj,
             "latent_prep: the projections' row of %d does not hold q at %d and the latent row at %d", ld_proj, q_off,
             down_off);
    IA_CHECK(slots == nullptr || (k_cache != nullptr && v_cache != nullptr), "latent_prep: slots without a cache");
    IA_CHECK(rd == 0 || (cos_t != nullptr && sin_t != nullptr), "latent_prep: a rotation without its tables");
    if (n == 0) return 0;
    if (rd == 0) cos_t = sin_t = nullptr;
    if (dtype == IA_F32)
        latent_prep_kernel<float><<<n, 256, 0, stream>>>((float*)q_out, (float*)k_cache, (float*)v_cache,
                                                         (const float*)proj, norm_w, cos_t, sin_t, slots, H, d, r, rank, rd,
                                                         q_off, down_off, ld_proj, page_size, eps, mag, interleaved, (const float*)qrows, ld_q);
    else
        latent_prep_kernel<bf16_t><<<n, 256, 0, stream>>>((bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache,
                                                          (const bf16_t*)proj, norm_w, cos_t, sin_t, slots, H, d, r, rank,
                                                          rd, q_off, down_off, ld_proj, page_size, eps, mag, interleaved, (const bf16_t*)qrows, ld_q) ;
    IA_LAUNCH_CHECK("latent_prep");
    return 0;
}

// ---- the RMS norm of a slice of wider rows: out[t][j] = x[t][x_off + j] / sqrt(mean_j x^2 + eps) * w[j] -----------------------------
// (a low-rank row that shares one product with its neighbours, normed on its way to the product that reads it)
template <typename T>
__global__ __launch_bounds__(256) void norm_slice_kernel(T* __restrict__ out, const T* __restrict__ x, long long x_ld, int x_off,
                                                         const float* __restrict__ w, float eps, int cols) {
    __shared__ float scratch[16];
    const T* row = x + (long long)blockIdx.x * x_ld + x_off;
    float sq = 0.f;
    for (int j = threadIdx.x; j < cols; j += blockDim.x) {
        const float v = ld(row + j);
        sq = fmaf(v, v, sq);
    }
    const float rs = 1.0f / sqrtf(block_sum(sq, scratch) / (float)cols + eps);
    for (int j = threadIdx.x; j < cols; j += blockDim.x) st(out + (long long)blockIdx.x * cols + j, ld(row + j) * rs * w[j]);
}

extern "C" int ia_norm_slice(void* out, const void* x, long long x_ld, int x_off, const float* w, float eps, int rows, int cols,
                             int dtype, hipStream_t stream) {
    IA_CHECK(rows >= 0 && cols > 0 && x_off >= 0 && x_off + cols <= x_ld && w != nullptr, "norm_slice: rows=%d cols=%d at %d of %lld",
             rows, cols, x_off, x_ld);
    if (rows == 0) return 0;
    if (dtype == IA_F32) norm_slice_kernel<float><<<rows, 256, 0, stream>>>((float*)out, (const float*)x, x_ld, x_off, w, eps, cols);
    else if (dtype == IA_BF16) norm_slice_kernel<bf16_t><<<rows, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, x_ld, x_off, w, eps, cols);
    else IA_CHECK(false, "norm_slice: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("norm_slice");
    return 0;
}

// ---- a product with a matrix of its own for every head -------------------------------------------------------------
// out[t][h][j] = sum_i w[h][j][i] * x[t][h][i]   (j < n_out, i < k_in; w is [H, n_out, k_in])
// x[t][h] starts at x + t * x_ld + x_off + h * x_head, out[t][h] at out + t * o_ld + o_off + h * o_head.  `gate`
// (null or like out, starting at gate + t * g_ld + g_off + h * n_out): the result is multiplied by its sigmoid.
template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(256) void head_product_kernel(
    TO* __restrict__ out, const TX* __restrict__ x, const TW* __restrict__ w, const TX* __restrict__ gate, int n,
    int n_out, int k_in, long long x_ld, int x_off, int x_head, long long o_ld, int o_off, int o_head, long long g_ld,
    int g_off, int g_per_head) {
    __shared__ TileShared sh;
    const int h = blockIdx.z, row0 = blockIdx.y * IA_TM, col0 = blockIdx.x * IA_TN;
    float acc[2][4], acc2[2][4];
    const TX* xb = x + x_off + (long long)h * x_head;
    auto xrow = [&](int i) -> const TX* { return row0 + i < n ? xb + (long long)(row0 + i) * x_ld : nullptr; };
    const TW* wt = w + ((long long)h * n_out + col0) * k_in;
    tile_product<TX, TW, false>(acc, acc2, sh, xrow, wt, wt, n_out - col0, k_in, k_in);
    const int ty = threadIdx.x >> 4, tx = threadIdx.x & 15;
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        const int t = row0 + 2 * ty + a;
        if (t >= n) continue;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int j = col0 + 4 * tx + b;
            if (j >= n_out) continue;
            float v = acc[a][b];
            if (gate != nullptr) {
                const float g = ld(gate + (long long)t * g_ld + g_off + (g_per_head ? h : (long long)h * n_out + j));
                v = v / (1.0f + expf(-g));
            }
            st(out + (long long)t * o_ld + o_off + (long long)h * o_head + j, v);
        }
    }
}

// The same on the matrix cores: bfloat16 rows and matrices, k_in and every offset a multiple of 8.
template <typename TO, int RT, int FT, int KC>
__global__ __launch_bounds__(256) void head_product_mfma_kernel(
    TO* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, const bf16_t* __restrict__ gate, int n,
    int n_out, int k_in, long long x_ld, int x_off, int x_head, long long o_ld, int o_off, int o_head, long long g_ld,
    int g_off, int g_per_head) {
    using Tile = TileMfma<RT, FT, KC, false>;
    __shared__ typename Tile::Shared sh;
    const int h = blockIdx.z, row0 = blockIdx.y * Tile::ROWS, col0 = blockIdx.x * Tile::FEATURES;
    tm_f32x4 acc[FT][RT], unused[FT][RT];
    const bf16_t* xb = x + x_off + (long long)h * x_head;
    auto xrow = [&](int i) -> const bf16_t* { return row0 + i < n ? xb + (long long)(row0 + i) * x_ld : nullptr; };
    const bf16_t* wt = w + ((long long)h * n_out + col0) * k_in;
    Tile::product(acc, unused, sh, xrow, wt, wt, n_out - col0, k_in, k_in);
    Tile::each([&](int i, int f, int ft, int rt, int q) {
        const int t = row0 + i, j = col0 + f;
        if (t >= n || j >= n_out) return;
        float v = acc[ft][rt][q];
        if (gate != nullptr) {
            const float g = ld(gate + (long long)t * g_ld + g_off + (g_per_head ? h : (long long)h * n_out + j));
            v = v / (1.0f + expf(-g));
        }
        st(out + (long long)t * o_ld + o_off + (long long)h * o_head + j, v);
    });
}

// dtypes: 0 float32, 1 bfloat16 (x and gate share one).  Combinations built: x and w and out alike; 32-bit results of
// bfloat16 matrices with rows in either precision.  bfloat16 rows and matrices whose sizes and offsets are multiples of
// 8 run on the matrix cores, the rest on the vector units.
extern "C" int ia_head_product(void* out, const void* x, const void* w, const void* gate, int n, int H, int n_out,
                               int k_in, long long x_ld, int x_off, int x_head, long long o_ld, int o_off, int o_head,
                               long long g_ld, int g_off, int g_per_head, int x_dtype, int w_dtype, int out_dtype,
                               hipStream_t stream) {
    IA_CHECK(n >= 0 && H > 0 && n_out > 0 && k_in > 0, "head_product: bad sizes n=%d heads=%d out=%d in=%d", n, H, n_out,
             k_in);
    IA_CHECK(x_off >= 0 && o_off >= 0 && x_off + (long long)(H - 1) * x_head + k_in <= x_ld &&
                 o_off + (long long)(H - 1) * o_head + n_out <= o_ld,
             "head_product: the heads do not fit rows of %lld and %lld", x_ld, o_ld);
    IA_CHECK(gate == nullptr || (g_off >= 0 && g_off + (long long)H * (g_per_head ? 1 : n_out) <= g_ld), "head_product: the gate does not fit its row");
    IA_CHECK(H <= 65535, "head_product: %d heads are more than a grid takes", H);
    if (n == 0) return 0;
    const dim3 grid((n_out + IA_TN - 1) / IA_TN, (n + IA_TM - 1) / IA_TM, H);
#define IA_LAUNCH(TX, TW, TO)                                                                                        \
    head_product_kernel<TX, TW, TO><<<grid, 256, 0, stream>>>((TO*)out, (const TX*)x, (const TW*)w, (const TX*)gate, n, \
                                                              n_out, k_in, x_ld, x_off, x_head, o_ld, o_off, o_head,  \
                                                              g_ld, g_off, g_per_head)
    const bool cores = x_dtype == IA_BF16 && w_dtype == IA_BF16 && k_in % 8 == 0 && x_ld % 8 == 0 && x_off % 8 == 0 &&
                       x_head % 8 == 0 && tile_mfma_aligned(x) && tile_mfma_aligned(w);
    // many rows and wide heads: tiles of 64 rows x 128 features (every operand read serves more products)
    const bool large = n >= 64 && n_out >= 128;
    const dim3 big((n_out + 127) / 128, (n + 63) / 64, H);
#define IA_CORES(TO, RT, FT, KC, G)                                                                                            \
    head_product_mfma_kernel<TO, RT, FT, KC><<<G, 256, 0, stream>>>((TO*)out, (const bf16_t*)x, (const bf16_t*)w,                 \
                                                                    (const bf16_t*)gate, n, n_out, k_in, x_ld, x_off, x_head,    \
                                                                    o_ld, o_off, o_head, g_ld, g_off, g_per_head)
    if (cores && out_dtype == IA_BF16 && large) IA_CORES(bf16_t, 4, 2, 64, big);
    else if (cores && out_dtype == IA_BF16) IA_CORES(bf16_t, 2, 1, 64, grid);
    else if (cores && out_dtype == IA_F32 && large) IA_CORES(float, 4, 2, 64, big);
    else if (cores && out_dtype == IA_F32) IA_CORES(float, 2, 1, 64, grid);
    else if (x_dtype == IA_F32 && w_dtype == IA_F32 && out_dtype == IA_F32) IA_LAUNCH(float, float, float);
    else if (x_dtype == IA_BF16 && w_dtype == IA_BF16 && out_dtype == IA_BF16) IA_LAUNCH(bf16_t, bf16_t, bf16_t);
    else if (x_dtype == IA_F32 && w_dtype == IA_BF16 && out_dtype == IA_F32) IA_LAUNCH(float, bf16_t, float);
    else if (x_dtype == IA_BF16 && w_dtype == IA_BF16 && out_dtype == IA_F32) IA_LAUNCH(bf16_t, bf16_t, float);
    else {
        ia_set_error("head_product: no kernel for the dtypes x=%d w=%d out=%d", x_dtype, w_dtype, out_dtype);
        return 1;
    }
#undef IA_LAUNCH
#undef IA_CORES
    IA_LAUNCH_CHECK("head_product");
    return 0;
}
