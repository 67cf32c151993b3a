// Routed experts: a router scores every expert for a token, the `top` best are run and their outputs added up
// with the scores as weights.
//
//   route      a wave a token: router logits as 32-bit sums whatever row and matrix are stored in, scores = sigmoid
//              (or softmax), the top experts by score (ties: the lower index), weights = score * scale (optionally
//              renormalised over the chosen).
//   plan       one block: the (token, k) pairs ordered by expert, and a table of row tiles (expert, first pair, rows),
//              all on the device: the host never learns how many tokens an expert got.
//   gate_up    tile by tile: rows gathered by pair, act(gate, up) in the epilogue.
//   down       tile by tile: one 32-bit output row a pair; whoever adds the experts up takes the pairs of a token
//              in the order of k, so a token's sum does not depend on what else is in the batch.
#include "api.h"
#include "common.h"
#include "tile_fma.h"
#include "tile_mfma.h"

#define IA_MAX_EXPERTS 256
#define IA_MAX_TOP 16

enum { IA_SCORE_SIGMOID = 0, IA_SCORE_SOFTMAX = 1 };

// eight neighbouring values of a row as 32-bit floats
__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float (&v)[8]) {
    const uint4 a = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}

#define IA_ROUTE_WAVES 4        // waves of a token's block
#define IA_ROUTE_FEW_TOKENS 64 // up to this many tokens a step the blocks are too few to hide a wave's chain of loads
#define IA_ROUTE_SHARE 8        // experts whose sums a wave holds at a time: a block takes 32 experts a round (routers of 33 to 64
                                // outputs: 10, 12 or 16, so that one walk over the row serves them all)

// The logits: a block of four waves a token; in every round of 32 experts a wave takes eight.  A lane owns the features
// 8 lane + 512 i of the row and adds its products up in that order (32-bit multiply-adds), then the lanes' sums meet in a
// butterfly: an order that depends on the width alone.  The logits meet in shared memory and the first wave picks.
// VEC: the width is a multiple of 8 (16-byte loads); else element by element.
// WAVES: the block's waves.  A logit is one wave's walk over the row whatever SHARE and WAVES are, so neither changes a sum.
template <typename T, bool VEC, int SHARE = IA_ROUTE_SHARE, int WAVES = IA_ROUTE_WAVES>
__global__ __launch_bounds__(64 * WAVES) void route_kernel(int* __restrict__ sel, float* __restrict__ weight,
                                                                    const T* __restrict__ h, const T* __restrict__ wr, int n,
                                                                    int W, int E, int top, float scale, int score_fn,
                                                                    int renorm, const float* __restrict__ choice_bias,
                                                                    int gates, float* __restrict__ gate_out) {
    // E counts every row of the router's matrix: the last `gates` of them take no part in the choice; the sigmoid of
    // such a row's logit is handed out as it is (gate_out [n, gates]): a gate a token, formed like a router's logit.
    __shared__ float logits[IA_MAX_EXPERTS];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const T* row = h + (long long)t * W;
    for (int e0 = wave * SHARE; e0 < E; e0 += WAVES * SHARE) {
        float acc[SHARE];
#pragma unroll
        for (int j = 0; j < SHARE; ++j) acc[j] = 0.f;
        // (four rounds of loads under way at once: a round is a trip to the memory)
#pragma unroll 4
        for (int c0 = lane * 8; c0 < W; c0 += IA_WAVE * 8) {
            float x[8];
            if (VEC) {
                load8(row + c0, x);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) x[i] = c0 + i < W ? ld(row + c0 + i) : 0.f;
            }
#pragma unroll
            for (int j = 0; j < SHARE; ++j) {
                // (an expert beyond the last reads the last one's row: no branch stands between the loads)
                const T* w = wr + (long long)(e0 + j < E ? e0 + j : E - 1) * W + c0;
                float wv[8];
                if (VEC) {
                    load8(w, wv);
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) wv[i] = c0 + i < W ? ld(w + i) : 0.f;
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[j] = fmaf(x[i], wv[i], acc[j]);
            }
        }
#pragma unroll
        for (int j = 0; j < SHARE; ++j) {
            const float total = wave_sum(acc[j]);
            if (lane == 0 && e0 + j < E) logits[e0 + j] = total;
        }
    }
    __syncthreads();
    if (wave != 0) return;
    if (gates > 0) {
        E -= gates;
        for (int j = lane; j < gates; j += IA_WAVE) gate_out[(long long)t * gates + j] = 1.0f / (1.0f + expf(-logits[E + j]));
    }
    float z[IA_MAX_EXPERTS / IA_WAVE];             // expert e lives in lane e % 64, register e / 64
#pragma unroll
    for (int q = 0; q < IA_MAX_EXPERTS / IA_WAVE; ++q) {
        const int e = q * IA_WAVE + lane;
        z[q] = e < E ? logits[e] : -INFINITY;
    }
    float zmax = -INFINITY, denom = 1.f;
    if (score_fn == IA_SCORE_SOFTMAX) {
#pragma unroll
        for (int q = 0; q < IA_MAX_EXPERTS / IA_WAVE; ++q) zmax = fmaxf(zmax, z[q]);
        zmax = wave_max(zmax);
        float s = 0.f;
#pragma unroll
        for (int q = 0; q < IA_MAX_EXPERTS / IA_WAVE; ++q) s += z[q] > -INFINITY ? expf(z[q] - zmax) : 0.f;
        denom = wave_sum(s);
    }
    float total = 0.f, mine = 0.f;
    int mine_e = 0;
    if (choice_bias != nullptr) {
        // The choice goes by score + bias, the weights by the score alone: the scores are formed first, and the picking
        // walks the biased ones (of equal ones the lower index).
        float sc[IA_MAX_EXPERTS / IA_WAVE], key[IA_MAX_EXPERTS / IA_WAVE];
#pragma unroll
        for (int q = 0; q < IA_MAX_EXPERTS / IA_WAVE; ++q) {
            const int e = q * IA_WAVE + lane;
            sc[q] = e < E ? (score_fn == IA_SCORE_SOFTMAX ? expf(z[q] - zmax) / denom : 1.0f / (1.0f + expf(-z[q]))) : 0.f;
            key[q] = e < E ? sc[q] + choice_bias[e] : -INFINITY;
        }
        for (int k = 0; k < top; ++k) {
            float best = -INFINITY, best_s = 0.f;
            int best_e = 0x7fffffff;
#pragma unroll
            for (int q = 0; q < IA_MAX_EXPERTS / IA_WAVE; ++q)
                if (key[q] > best) { best = key[q]; best_e = q * IA_WAVE + lane; best_s = sc[q]; }
#pragma unroll
            for (int o = IA_WAVE / 2; o > 0; o >>= 1) {
                const float ob = __shfl_xor(best, o, IA_WAVE), os = __shfl_xor(best_s, o, IA_WAVE);
                const int oe = __shfl_xor(best_e, o, IA_WAVE);
                if (ob > best || (ob == best && oe < best_e)) { best = ob; best_e = oe; best_s = os; }
            }
#pragma unroll
            for (int q = 0; q < IA_MAX_EXPERTS / IA_WAVE; ++q)
                if (best_e == q * IA_WAVE + lane) key[q] = -INFINITY;
            total += best_s;
            if (lane == k) { mine = best_s; mine_e = best_e; }
        }
    } else
    for (int k = 0; k < top; ++k) {
        // every lane's best, then the wave's: the largest logit, of equal ones the lower index
        float best = -INFINITY;
        int best_e = 0x7fffffff;
#pragma unroll
        for (int q = 0; q < IA_MAX_EXPERTS / IA_WAVE; ++q)
            if (z[q] > best) { best = z[q]; best_e = q * IA_WAVE + lane; }
#pragma unroll
        for (int o = IA_WAVE / 2; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, IA_WAVE);
            const int oe = __shfl_xor(best_e, o, IA_WAVE);
            if (ob > best || (ob == best && oe < best_e)) { best = ob; best_e = oe; }
        }
#pragma unroll
        for (int q = 0; q < IA_MAX_EXPERTS / IA_WAVE; ++q)
            if (best_e == q * IA_WAVE + lane) z[q] = -INFINITY;
        const float s = score_fn == IA_SCORE_SOFTMAX ? expf(best - zmax) / denom : 1.0f / (1.0f + expf(-best));
        total += s;
        if (lane == k) { mine = s; mine_e = best_e; }
    }
    if (lane < top) {
        sel[(long long)t * top + lane] = mine_e;
        weight[(long long)t * top + lane] = (renorm ? mine / total : mine) * scale;
    }
}

// One block.  `order` [pairs]: the pairs grouped by expert; tiles: expert, first place in `order`, rows; meta[0]: tiles.
__global__ __launch_bounds__(1024) void route_plan_kernel(int* __restrict__ order, int* __restrict__ tile_expert,
                                                          int* __restrict__ tile_first, int* __restrict__ tile_rows,
                                                          int* __restrict__ meta, const int* __restrict__ sel, int pairs,
                                                          int E, int tile) {
    __shared__ int count[IA_MAX_EXPERTS], first[IA_MAX_EXPERTS], tile0[IA_MAX_EXPERTS], cursor[IA_MAX_EXPERTS];
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = cursor[e] = 0;
    __syncthreads();
    // (a choice of E or beyond names no expert with weights: such a pair gets no place and no tile)
    for (int p = threadIdx.x; p < pairs; p += blockDim.x)
        if (sel[p] < E) atomicAdd(&count[sel[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, tiles = 0;
        for (int e = 0; e < E; ++e) {
            first[e] = at;
            tile0[e] = tiles;
            at += count[e];
            tiles += (count[e] + tile - 1) / tile;
        }
        meta[0] = tiles;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        const int tiles = (count[e] + tile - 1) / tile;
        for (int i = 0; i < tiles; ++i) {
            tile_expert[tile0[e] + i] = e;
            tile_first[tile0[e] + i] = first[e] + i * tile;
            tile_rows[tile0[e] + i] = min(tile, count[e] - i * tile);
        }
    }
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        const int e = sel[p];
        if (e < E) order[first[e] + atomicAdd(&cursor[e], 1)] = p;
    }
}

// act[place][j] = g' * sigmoid(alpha g') * (u' + 1), g' = min(gate_j . x, limit), u' = clamp(up_j . x, -limit, limit);
// x = h[pair / top] (times in_weight[pair], where given: 32-bit, one a pair).  w_gu [E][2 ff][W]: an expert's gate rows, then its up rows.
template <typename T>
__global__ __launch_bounds__(256) void experts_gate_up_kernel(T* __restrict__ act, const T* __restrict__ h,
                                                              const T* __restrict__ w_gu, const int* __restrict__ order,
                                                              const int* __restrict__ tile_expert,
                                                              const int* __restrict__ tile_first,
                                                              const int* __restrict__ tile_rows,
                                                              const int* __restrict__ meta, int top, int W, int ff,
                                                              float limit, float alpha, const float* __restrict__ in_weight) {
    __shared__ TileShared sh;
    const int tile = blockIdx.y;
    if (tile >= meta[0]) return;
    const int e = tile_expert[tile], first = tile_first[tile], rows = tile_rows[tile], col0 = blockIdx.x * IA_TN;
    float g[2][4], u[2][4];
    auto xrow = [&](int i) -> const T* { return i < rows ? h + (long long)(order[first + i] / top) * W : nullptr; };
    const T* wg = w_gu + ((long long)e * 2 * ff + col0) * W;
    tile_product<T, T, true>(g, u, sh, xrow, wg, wg + (long long)ff * W, ff - col0, W, W);
    const int ty = threadIdx.x >> 4, tx = threadIdx.x & 15;
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        const int i = 2 * ty + a;
        if (i >= rows) continue;
        // (in_weight: the pair's weight is a factor on the expert's INPUT, hence on both sums ahead of the limits)
        const float wi = in_weight != nullptr ? in_weight[order[first + i]] : 1.0f;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int j = col0 + 4 * tx + b;
            if (j >= ff) continue;
            const float gv = fminf(g[a][b] * wi, limit), uv = fminf(fmaxf(u[a][b] * wi, -limit), limit);
            st(act + (long long)(first + i) * ff + j, gv / (1.0f + expf(-alpha * gv)) * (uv + 1.0f));
        }
    }
}

// y[pair][c] = down_c . act[place]   (32-bit rows, one a pair)
template <typename T>
__global__ __launch_bounds__(256) void experts_down_kernel(float* __restrict__ y, const T* __restrict__ act,
                                                           const T* __restrict__ w_down, const int* __restrict__ order,
                                                           const int* __restrict__ tile_expert,
                                                           const int* __restrict__ tile_first,
                                                           const int* __restrict__ tile_rows,
                                                           const int* __restrict__ meta, int W, int ff) {
    __shared__ TileShared sh;
    const int tile = blockIdx.y;
    if (tile >= meta[0]) return;
    const int e = tile_expert[tile], first = tile_first[tile], rows = tile_rows[tile], col0 = blockIdx.x * IA_TN;
    float acc[2][4], unused[2][4];
    auto xrow = [&](int i) -> const T* { return i < rows ? act + (long long)(first + i) * ff : nullptr; };
    const T* wd = w_down + ((long long)e * W + col0) * ff;
    tile_product<T, T, false>(acc, unused, sh, xrow, wd, wd, W - col0, ff, ff);
    const int ty = threadIdx.x >> 4, tx = threadIdx.x & 15;
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        const int i = 2 * ty + a;
        if (i >= rows) continue;
        const long long pair = order[first + i];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int c = col0 + 4 * tx + b;
            if (c < W) y[pair * W + c] = acc[a][b];
        }
    }
}

// The same two products on the matrix cores (bfloat16; widths in steps of 8) over weights stored as tiles (see
// tile_mfma.h): w_gu [E][2][ceil(ff / 64)][ceil(W / 64)][64][64], w_down [E][ceil(W / 64)][ceil(ff / 64)][64][64].
template <int RT, int FT>
__global__ __launch_bounds__(256) void experts_gate_up_mfma_kernel(bf16_t* __restrict__ act, const bf16_t* __restrict__ h,
                                                                   const bf16_t* __restrict__ w_gu,
                                                                   const int* __restrict__ order,
                                                                   const int* __restrict__ tile_expert,
                                                                   const int* __restrict__ tile_first,
                                                                   const int* __restrict__ tile_rows,
                                                                   const int* __restrict__ meta, int top, int W, int ff,
                                                                   float limit, float alpha, const float* __restrict__ in_weight) {
    using Tile = TileMfma<RT, FT, 64, true>;
    __shared__ typename Tile::Shared sh;
    const int tile = blockIdx.y;
    if (tile >= meta[0]) return;
    const int e = tile_expert[tile], first = tile_first[tile], rows = tile_rows[tile], col0 = blockIdx.x * Tile::FEATURES;
    const int fbs = (ff + 63) / 64, chunks = (W + 63) / 64;
    tm_f32x4 g[FT][RT], u[FT][RT];
    auto xrow = [&](int i) -> const bf16_t* { return i < rows ? h + (long long)(order[first + i] / top) * W : nullptr; };
    const long long matrix = (long long)fbs * chunks * 4096;
    const bf16_t* wg = w_gu + (long long)e * 2 * matrix + (long long)(col0 / 64) * chunks * 4096;
    Tile::product_tiled(g, u, sh, xrow, wg, wg + matrix, fbs - col0 / 64, chunks, W);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int i = 16 * rt + (lane & 15);
        const float wi = in_weight != nullptr && i < rows ? in_weight[order[first + i]] : 1.0f;
#pragma unroll
        for (int ft = 0; ft < FT; ++ft) {
            const int j0 = col0 + 16 * (wave * FT + ft) + 4 * (lane >> 4);
            const tm_f32x4 gq = g[ft][rt], uq = u[ft][rt];
            const float gs[4] = {gq[0], gq[1], gq[2], gq[3]}, us[4] = {uq[0], uq[1], uq[2], uq[3]};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (i >= rows || j0 + q >= ff) continue;
                const float gv = fminf(gs[q] * wi, limit), uv = fminf(fmaxf(us[q] * wi, -limit), limit);
                st(act + (long long)(first + i) * ff + j0 + q, gv / (1.0f + expf(-alpha * gv)) * (uv + 1.0f));
            }
        }
    }
}

template <int RT, int FT>
__global__ __launch_bounds__(256) void experts_down_mfma_kernel(float* __restrict__ y, const bf16_t* __restrict__ act,
                                                                const bf16_t* __restrict__ w_down,
                                                                const int* __restrict__ order,
                                                                const int* __restrict__ tile_expert,
                                                                const int* __restrict__ tile_first,
                                                                const int* __restrict__ tile_rows,
                                                                const int* __restrict__ meta, int W, int ff) {
    using Tile = TileMfma<RT, FT, 64, false>;
    __shared__ typename Tile::Shared sh;
    const int tile = blockIdx.y;
    if (tile >= meta[0]) return;
    const int e = tile_expert[tile], first = tile_first[tile], rows = tile_rows[tile], col0 = blockIdx.x * Tile::FEATURES;
    const int fbs = (W + 63) / 64, chunks = (ff + 63) / 64;
    tm_f32x4 acc[FT][RT], unused[FT][RT];
    auto xrow = [&](int i) -> const bf16_t* { return i < rows ? act + (long long)(first + i) * ff : nullptr; };
    const bf16_t* wd = w_down + ((long long)e * fbs + col0 / 64) * chunks * 4096;
    Tile::product_tiled(acc, unused, sh, xrow, wd, wd, fbs - col0 / 64, chunks, ff);
    Tile::each([&](int i, int f, int ft, int rt, int q) {
        const int c = col0 + f;
        if (i < rows && c < W) y[(long long)order[first + i] * W + c] = acc[ft][rt][q];
    });
}

// choice_bias: null, or [E] 32-bit values added to the scores for the choice only (the weights are the scores themselves)
extern "C" int ia_route(int* sel, float* weight, const void* h, const void* router, int n, int W, int E, int top,
                        float scale, int score_fn, int renorm, const float* choice_bias, int gates, float* gate_out,
                        int dtype, hipStream_t stream) {
    // E: the router's outputs that can be chosen; the matrix holds `gates` more rows behind them (see the kernel)
    IA_CHECK(gates >= 0 && (gates == 0 || gate_out != nullptr), "route: %d gate rows need a place for their values", gates);
    IA_CHECK(n >= 0 && W > 0 && E >= 1 && E + gates <= IA_MAX_EXPERTS && top >= 1 && top <= E && top <= IA_MAX_TOP,
             "route: n=%d width=%d experts=%d and %d gate rows (up to %d) top=%d (up to %d)", n, W, E, gates, IA_MAX_EXPERTS, top, IA_MAX_TOP);
    E += gates;
    IA_CHECK(score_fn == IA_SCORE_SIGMOID || score_fn == IA_SCORE_SOFTMAX, "route: unknown score function %d", score_fn);
    if (n == 0) return 0;
    const bool vec = W % 8 == 0 && tile_mfma_aligned(h) && tile_mfma_aligned(router);
#define IA_ROUTE_SW(T, V, S, WV) route_kernel<T, V, S, WV><<<n, 64 * WV, 0, stream>>>(sel, weight, (const T*)h, (const T*)router, n, W, E, top, scale, score_fn, renorm, choice_bias, gates, gate_out)
#define IA_ROUTE_S(T, V, S) IA_ROUTE_SW(T, V, S, IA_ROUTE_WAVES)
    // (up to 32 outputs: 8 a wave; up to 64: as many a wave as take them all in one walk over the row.  A step of few
    // tokens has few blocks, and a wave's walk is a chain of trips to the memory: sixteen waves a token then, each with
    // as few outputs as share them all out)
#define IA_ROUTE(T, V) do { if (n <= IA_ROUTE_FEW_TOKENS && E > 8) { \
            if (E <= 16) IA_ROUTE_SW(T, V, 1, 16); else if (E <= 32) IA_ROUTE_SW(T, V, 2, 16); \
            else if (E <= 48) IA_ROUTE_SW(T, V, 3, 16); else if (E <= 64) IA_ROUTE_SW(T, V, 4, 16); else IA_ROUTE_SW(T, V, 8, 16); } \
        else if (E <= 32 || E > 64) IA_ROUTE_S(T, V, 8); else if (E <= 40) IA_ROUTE_S(T, V, 10); \
        else if (E <= 48) IA_ROUTE_S(T, V, 12); else IA_ROUTE_S(T, V, 16); } while (0)
    if (dtype == IA_F32) { if (vec) IA_ROUTE(float, true); else IA_ROUTE(float, false); }
    else { if (vec) IA_ROUTE(bf16_t, true); else IA_ROUTE(bf16_t, false); }
#undef IA_ROUTE_SW
#undef IA_ROUTE_S
#undef IA_ROUTE
    IA_LAUNCH_CHECK("route");
    return 0;
}

// The most tiles of `tile` rows that `pairs` pairs over E experts can make: the grids of the two products.
static int route_tiles(int pairs, int E, int tile) { return (pairs + tile - 1) / tile + (E < pairs ? E : pairs); }
extern "C" int ia_route_tiles(int pairs, int E) { return route_tiles(pairs, E, IA_TM); }

// tile: rows of a tile, 32 (every kernel) or 64 or 128 (the matrix cores' large shapes, for many rows an expert)
extern "C" int ia_route_plan(int* order, int* tile_expert, int* tile_first, int* tile_rows, int* meta, const int* sel,
                             int pairs, int E, int tile, hipStream_t stream) {
    IA_CHECK(pairs >= 0 && E >= 1 && E <= IA_MAX_EXPERTS && (tile == 32 || tile == 64 || tile == 128), "route_plan: pairs=%d experts=%d tile=%d",
             pairs, E, tile);
    route_plan_kernel<<<1, 1024, 0, stream>>>(order, tile_expert, tile_first, tile_rows, meta, sel, pairs, E, tile);
    IA_LAUNCH_CHECK("route_plan");
    return 0;
}

extern "C" int ia_experts_gate_up(void* act, const void* h, const void* w_gu, const int* order, const int* tile_expert,
                                  const int* tile_first, const int* tile_rows, const int* meta, int pairs, int E, int top,
                                  int W, int ff, float limit, float alpha, int tile, int tiled, const float* in_weight, int dtype,
                                  hipStream_t stream) {
    IA_CHECK(pairs >= 0 && W > 0 && ff > 0 && top >= 1 && limit > 0.f && (tile == 32 || tile == 64 || tile == 128), "experts_gate_up: bad sizes");
    if (pairs == 0) return 0;
    IA_CHECK(!tiled || (dtype == IA_BF16 && W % 8 == 0 && tile_mfma_aligned(h) && tile_mfma_aligned(w_gu)),
             "experts_gate_up: weights stored as tiles are the matrix cores' (bfloat16, widths in steps of 8)");
    IA_CHECK(tile == 32 || tiled, "experts_gate_up: tiles of 64 or 128 rows go with weights stored as tiles");
    const int features = tile == 32 ? 64 : 128;
    const dim3 grid((ff + features - 1) / features, route_tiles(pairs, E, tile));
    IA_CHECK(grid.y <= 65535, "experts_gate_up: %u row tiles are more than a grid takes", grid.y);
    if (tiled && tile == 128)
        experts_gate_up_mfma_kernel<8, 2><<<grid, 256, 0, stream>>>((bf16_t*)act, (const bf16_t*)h, (const bf16_t*)w_gu, order,
                                                                    tile_expert, tile_first, tile_rows, meta, top, W, ff, limit, alpha, in_weight);
    else if (tiled && tile == 64)
        experts_gate_up_mfma_kernel<4, 2><<<grid, 256, 0, stream>>>((bf16_t*)act, (const bf16_t*)h, (const bf16_t*)w_gu, order,
                                                                    tile_expert, tile_first, tile_rows, meta, top, W, ff, limit, alpha, in_weight);
    else if (tiled)
        experts_gate_up_mfma_kernel<2, 1><<<grid, 256, 0, stream>>>((bf16_t*)act, (const bf16_t*)h, (const bf16_t*)w_gu, order,
                                                                    tile_expert, tile_first, tile_rows, meta, top, W, ff, limit, alpha, in_weight);
    else if (dtype == IA_F32)
        experts_gate_up_kernel<float><<<grid, 256, 0, stream>>>((float*)act, (const float*)h, (const float*)w_gu, order,
                                                                tile_expert, tile_first, tile_rows, meta, top, W, ff, limit, alpha, in_weight);
    else
        experts_gate_up_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)act, (const bf16_t*)h, (const bf16_t*)w_gu, order,
                                                                 tile_expert, tile_first, tile_rows, meta, top, W, ff, limit, alpha, in_weight);
    IA_LAUNCH_CHECK("experts_gate_up");
    return 0;
}

extern "C" int ia_experts_down(float* y, const void* act, const void* w_down, const int* order, const int* tile_expert,
                               const int* tile_first, const int* tile_rows, const int* meta, int pairs, int E, int W,
                               int ff, int tile, int tiled, int dtype, hipStream_t stream) {
    IA_CHECK(pairs >= 0 && W > 0 && ff > 0 && (tile == 32 || tile == 64 || tile == 128), "experts_down: bad sizes");
    if (pairs == 0) return 0;
    IA_CHECK(!tiled || (dtype == IA_BF16 && ff % 8 == 0 && tile_mfma_aligned(act) && tile_mfma_aligned(w_down)),
             "experts_down: weights stored as tiles are the matrix cores' (bfloat16, widths in steps of 8)");
    IA_CHECK(tile == 32 || tiled, "experts_down: tiles of 64 or 128 rows go with weights stored as tiles");
    const int features = tile == 32 ? 64 : 128;
    const dim3 grid((W + features - 1) / features, route_tiles(pairs, E, tile));
    IA_CHECK(grid.y <= 65535, "experts_down: %u row tiles are more than a grid takes", grid.y);
    if (tiled && tile == 128)
        experts_down_mfma_kernel<8, 2><<<grid, 256, 0, stream>>>(y, (const bf16_t*)act, (const bf16_t*)w_down, order, tile_expert,
                                                                 tile_first, tile_rows, meta, W, ff);
    else if (tiled && tile == 64)
        experts_down_mfma_kernel<4, 2><<<grid, 256, 0, stream>>>(y, (const bf16_t*)act, (const bf16_t*)w_down, order, tile_expert,
                                                                 tile_first, tile_rows, meta, W, ff);
    else if (tiled)
        experts_down_mfma_kernel<2, 1><<<grid, 256, 0, stream>>>(y, (const bf16_t*)act, (const bf16_t*)w_down, order, tile_expert,
                                                                 tile_first, tile_rows, meta, W, ff);
    else if (dtype == IA_F32)
        experts_down_kernel<float><<<grid, 256, 0, stream>>>(y, (const float*)act, (const float*)w_down, order, tile_expert,
                                                             tile_first, tile_rows, meta, W, ff);
    else
        experts_down_kernel<bf16_t><<<grid, 256, 0, stream>>>(y, (const bf16_t*)act, (const bf16_t*)w_down, order, tile_expert,
                                                              tile_first, tile_rows, meta, W, ff);
    IA_LAUNCH_CHECK("experts_down");
    return 0;
}
