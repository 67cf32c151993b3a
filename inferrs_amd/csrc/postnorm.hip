// A residual stream kept in 32-bit that is normed AFTER every sum:
//     x <- rmsnorm(alpha x + y (+ sum_k w_k r_k) (+ y2)) * w
// ONE kernel does what stands behind a sub-layer: it scales the stream, adds the sub-layer's output (a dense one, the
// rows of routed experts with their weights, a second dense one beside them: every one optional), norms the sum and
// writes it back, in 32-bit and (optionally) once more in the products' precision for the next sub-layer to read.
// A routed row whose expert index is `real_experts` or more stands for an expert that hands its input on: the stream's
// own row takes its place.  A block owns a row; the sum and the sum of squares are 32-bit.  With `rows` the kernel reads
// the named rows only and leaves the stream alone (the model's end: the wanted rows through the final norm).
//
// Beside it: the embedding's rows scaled into such a stream, a sigmoid gate on rows in place, the clamped gate of
// experts on a dense [gate | up] product, and a factor on 32-bit logits.
#include "api.h"
#include "common.h"

#define PN_MAX_TOP 16

// An output that is still split along the k of its product, [splits, n, W]: the splits' sums added up in their order.
template <typename T>
__device__ __forceinline__ float pn_sum_splits(const T* p, int splits, long long stride) {
    float t = ld(p);
    for (int s = 1; s < splits; ++s) t += ld(p + s * stride);
    return t;
}

template <typename TY, typename TH>
__global__ __launch_bounds__(1024) void postnorm_step_kernel(
    float* __restrict__ x, float alpha, const TY* __restrict__ y, const TY* __restrict__ y2, int y_splits, int y2_splits,
    long long split_stride, const float* __restrict__ routed, const float* __restrict__ routed_w,
    const int* __restrict__ sel, int top, int real_experts, const float* __restrict__ w, float eps, TH* __restrict__ h,
    const int* __restrict__ rows, int W) {
    extern __shared__ float pn_row[];            // [W]
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int row = rows != nullptr ? rows[r] : r;
    float* xr = x + (long long)row * W;
    float wk[PN_MAX_TOP];
    bool own[PN_MAX_TOP];
#pragma unroll
    for (int k = 0; k < PN_MAX_TOP; ++k) {
        const bool on = routed != nullptr && k < top;
        wk[k] = on ? routed_w[(long long)row * top + k] : 0.f;
        own[k] = on && sel != nullptr && sel[(long long)row * top + k] >= real_experts;
    }
    float sq = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float xv = xr[c];
        float v = alpha * xv;
        if (y != nullptr) v += pn_sum_splits(y + (long long)row * W + c, y_splits, split_stride);
        if (routed != nullptr) {
#pragma unroll
            for (int k = 0; k < PN_MAX_TOP; ++k)
                if (k < top) v = fmaf(wk[k], own[k] ? xv : routed[((long long)row * top + k) * W + c], v);
        }
        if (y2 != nullptr) v += pn_sum_splits(y2 + (long long)row * W + c, y2_splits, split_stride);
        pn_row[c] = v;
        sq = fmaf(v, v, sq);
    }
    const float rs = 1.0f / sqrtf(block_sum(sq, scratch) / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float v = pn_row[c] * rs * w[c];
        if (rows == nullptr) xr[c] = v;
        if (h != nullptr) st(h + (long long)r * W + c, v);
    }
}

// The same for widths in steps of 8 up to 8 * PN_VEC_ITERS * the block's threads: a thread owns eight neighbouring
// features a round (16- and 32-byte accesses), the row's sum stays in its registers between the two passes, and nothing
// goes through shared memory but the sum of squares.  The arithmetic of a feature is that of the kernel above.
#define PN_VEC_ITERS 4

__device__ __forceinline__ void pn_load8(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void pn_load8(const bf16_t* p, float (&v)[8]) {
    const uint4 a = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}
__device__ __forceinline__ void pn_store8(float* p, const float (&v)[8]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void pn_store8(bf16_t* p, const float (&v)[8]) {
    *reinterpret_cast<uint4*>(p) = make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]),
                                              pack_bf16x2(v[6], v[7]));
}

template <typename T>
__device__ __forceinline__ void pn_load8_splits(const T* p, int splits, long long stride, float (&t)[8]) {
    pn_load8(p, t);
    for (int s = 1; s < splits; ++s) {
        float u[8];
        pn_load8(p + s * stride, u);
#pragma unroll
        for (int i = 0; i < 8; ++i) t[i] += u[i];
    }
}

template <typename TY, typename TH>
__global__ __launch_bounds__(1024) void postnorm_step_vec_kernel(
    float* __restrict__ x, float alpha, const TY* __restrict__ y, const TY* __restrict__ y2, int y_splits, int y2_splits,
    long long split_stride, const float* __restrict__ routed, const float* __restrict__ routed_w,
    const int* __restrict__ sel, int top, int real_experts, const float* __restrict__ w, float eps, TH* __restrict__ h,
    const int* __restrict__ rows, int W) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int row = rows != nullptr ? rows[r] : r;
    float* xr = x + (long long)row * W;
    float wk[PN_MAX_TOP];
    bool own[PN_MAX_TOP];
#pragma unroll
    for (int k = 0; k < PN_MAX_TOP; ++k) {
        const bool on = routed != nullptr && k < top;
        wk[k] = on ? routed_w[(long long)row * top + k] : 0.f;
        own[k] = on && sel != nullptr && sel[(long long)row * top + k] >= real_experts;
    }
    float v[PN_VEC_ITERS][8];
    float sq = 0.f;
#pragma unroll
    for (int it = 0; it < PN_VEC_ITERS; ++it) {
        const int c = (it * blockDim.x + threadIdx.x) * 8;
        if (c >= W) continue;
        float xv[8], t[8];
        pn_load8(xr + c, xv);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[it][i] = alpha * xv[i];
        if (y != nullptr) {
            pn_load8_splits(y + (long long)row * W + c, y_splits, split_stride, t);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[it][i] += t[i];
        }
        if (routed != nullptr) {
#pragma unroll
            for (int k = 0; k < PN_MAX_TOP; ++k) {
                if (k >= top) break;
                if (own[k]) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) v[it][i] = fmaf(wk[k], xv[i], v[it][i]);
                } else {
                    pn_load8(routed + ((long long)row * top + k) * W + c, t);
#pragma unroll
                    for (int i = 0; i < 8; ++i) v[it][i] = fmaf(wk[k], t[i], v[it][i]);
                }
            }
        }
        if (y2 != nullptr) {
            pn_load8_splits(y2 + (long long)row * W + c, y2_splits, split_stride, t);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[it][i] += t[i];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) sq = fmaf(v[it][i], v[it][i], sq);
    }
    const float rs = 1.0f / sqrtf(block_sum(sq, scratch) / (float)W + eps);
#pragma unroll
    for (int it = 0; it < PN_VEC_ITERS; ++it) {
        const int c = (it * blockDim.x + threadIdx.x) * 8;
        if (c >= W) continue;
        float wv[8], o[8];
        pn_load8(w + c, wv);
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = v[it][i] * rs * wv[i];
        if (rows == nullptr) pn_store8(xr + c, o);
        if (h != nullptr) pn_store8(h + (long long)r * W + c, o);
    }
}

// y_dtype: precision of y and y2; h_dtype: of h.  0 float32, 1 bfloat16.  y_splits, y2_splits: 1, or the splits of a product
// that is still split along its k ([splits, n, W], 32-bit), which the kernel adds up in their order.
extern "C" int ia_postnorm_step(float* x, float alpha, const void* y, const void* y2, int y_splits, int y2_splits,
                                const float* routed, const float* routed_w, const int* sel, int top, int real_experts,
                                const float* w, float eps, void* h, const int* rows, int n, int W, int y_dtype, int h_dtype,
                                hipStream_t stream) {
    IA_CHECK(n >= 0 && W > 0 && w != nullptr, "postnorm_step: n=%d width=%d, and the norm's weight", n, W);
    IA_CHECK((size_t)W * sizeof(float) <= 60 * 1024, "postnorm_step: width %d does not fit shared memory", W);
    IA_CHECK(routed == nullptr || (routed_w != nullptr && top >= 1 && top <= PN_MAX_TOP),
             "postnorm_step: routed rows come with their weights, up to %d a row (top=%d)", PN_MAX_TOP, top);
    IA_CHECK(rows == nullptr || h != nullptr, "postnorm_step: a row list leaves the stream alone, so it needs an output");
    IA_CHECK(y_splits >= 1 && y2_splits >= 1 && ((y_splits == 1 && y2_splits == 1) || (y_dtype == IA_F32 && rows == nullptr)),
             "postnorm_step: outputs in %d and %d splits are 32-bit and cover every row", y_splits, y2_splits);
    if (n == 0) return 0;
    const long long split_stride = (long long)n * W;
    const uintptr_t ptrs = (uintptr_t)x | (uintptr_t)y | (uintptr_t)y2 | (uintptr_t)routed | (uintptr_t)w | (uintptr_t)h;
    if (W % 8 == 0 && (ptrs & 15) == 0 && W <= 8 * PN_VEC_ITERS * 1024) {
        // as many threads as the row has pieces of eight, in whole waves, a round or more each
        int threads = (W / 8 + 63) / 64 * 64;
        if (threads > 256) threads = (W / 8 + 2 * 64 - 1) / (2 * 64) * 64;          // two rounds a thread
        if (threads > 512) threads = (W / 8 + PN_VEC_ITERS * 64 - 1) / (PN_VEC_ITERS * 64) * 64;
#define IA_LAUNCH_VEC(TY, TH)                                                                                          \
    postnorm_step_vec_kernel<TY, TH><<<n, threads, 0, stream>>>(x, alpha, (const TY*)y, (const TY*)y2, y_splits, y2_splits, \
                                                                split_stride, routed, routed_w, sel, top, real_experts, w, eps, \
                                                                (TH*)h, rows, W)
        if (y_dtype == IA_F32 && h_dtype == IA_F32) { IA_LAUNCH_VEC(float, float); }
        else if (y_dtype == IA_F32) { IA_LAUNCH_VEC(float, bf16_t); }
        else if (h_dtype == IA_F32) { IA_LAUNCH_VEC(bf16_t, float); }
        else { IA_LAUNCH_VEC(bf16_t, bf16_t); }
#undef IA_LAUNCH_VEC
        IA_LAUNCH_CHECK("postnorm_step");
        return 0;
    }
    const int threads = W >= 4096 ? 1024 : W >= 1024 ? 512 : 256;
    const size_t shm = (size_t)W * sizeof(float);
#define IA_LAUNCH(TY, TH)                                                                                            \
    postnorm_step_kernel<TY, TH><<<n, threads, shm, stream>>>(x, alpha, (const TY*)y, (const TY*)y2, y_splits, y2_splits, \
                                                              split_stride, routed, routed_w, sel, top, real_experts, w, eps, \
                                                              (TH*)h, rows, W)
    if (y_dtype == IA_F32 && h_dtype == IA_F32) { IA_LAUNCH(float, float); }
    else if (y_dtype == IA_F32) { IA_LAUNCH(float, bf16_t); }
    else if (h_dtype == IA_F32) { IA_LAUNCH(bf16_t, float); }
    else { IA_LAUNCH(bf16_t, bf16_t); }
#undef IA_LAUNCH
    IA_LAUNCH_CHECK("postnorm_step");
    return 0;
}

// ---- the embedding's rows, scaled, as a 32-bit stream (and once more in the products' precision) ---------------------
template <typename T>
__global__ void embed_scaled_kernel(float* __restrict__ out, T* __restrict__ h, const T* __restrict__ table,
                                    const int* __restrict__ ids, int hidden, int vocab, float scale) {
    const int row = blockIdx.x;
    const int id = ids[row];
    const bool ok = id >= 0 && id < vocab;
    const T* src = table + (size_t)(ok ? id : 0) * hidden;
    for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
        const float v = ok ? ld(src + c) * scale : 0.f;
        out[(size_t)row * hidden + c] = v;
        if (h != nullptr) st(h + (size_t)row * hidden + c, v);
    }
}

extern "C" int ia_embed_gather_scaled(float* out, void* h, const void* table, const int* ids, int n, int hidden, int vocab,
                                      float scale, int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && hidden > 0 && vocab > 0, "embed_gather_scaled: bad sizes n=%d hidden=%d vocab=%d", n, hidden, vocab);
    if (n == 0) return 0;
    const int block = hidden >= 1024 ? 256 : 64;
    if (dtype == IA_F32)
        embed_scaled_kernel<float><<<n, block, 0, stream>>>(out, (float*)h, (const float*)table, ids, hidden, vocab, scale);
    else if (dtype == IA_BF16)
        embed_scaled_kernel<bf16_t><<<n, block, 0, stream>>>(out, (bf16_t*)h, (const bf16_t*)table, ids, hidden, vocab, scale);
    else
        IA_CHECK(false, "embed_gather_scaled: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("embed_gather_scaled");
    return 0;
}

// ---- a[row][c] *= sigmoid(g[row][g_off + c]) in place ------------------------------------------------------------------
template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ a, const T* __restrict__ g, int cols, int g_ld, int g_off, int group,
                                    size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t row = i / cols;
        const int c = (int)(i - row * cols);
        const float z = ld(g + row * g_ld + g_off + c / group);
        st(a + i, ld(a + i) / (1.0f + expf(-z)));
    }
}

// bfloat16 rows whose length, pitch and offset are multiples of 8: eight values a thread, 16-byte accesses
__global__ void sigmoid_gate_bf16_vec_kernel(bf16_t* __restrict__ a, const bf16_t* __restrict__ g, int cols, int g_ld, int g_off,
                                             size_t total_vecs) {
    const int vecs_per_row = cols / 8;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total_vecs; i += (size_t)gridDim.x * blockDim.x) {
        const size_t row = i / vecs_per_row;
        const int c = (int)(i - row * vecs_per_row) * 8;
        const uint4 ar = *(const uint4*)(a + row * cols + c);
        const uint4 gr = *(const uint4*)(g + row * g_ld + g_off + c);
        const uint32_t aw[4] = {ar.x, ar.y, ar.z, ar.w}, gw[4] = {gr.x, gr.y, gr.z, gr.w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float a0 = __uint_as_float(aw[j] << 16), a1 = __uint_as_float(aw[j] & 0xffff0000u);
            const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
            o[j] = pack_bf16x2(a0 / (1.0f + expf(-g0)), a1 / (1.0f + expf(-g1)));
        }
        *(uint4*)(a + row * cols + c) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// The same where `group` columns (a multiple of 8) share one gate value: eight values a thread and one sigmoid
__global__ void sigmoid_gate_group_bf16_vec_kernel(bf16_t* __restrict__ a, const bf16_t* __restrict__ g, int cols, int g_ld,
                                                   int g_off, int group, size_t total_vecs) {
    const int vecs_per_row = cols / 8;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total_vecs; i += (size_t)gridDim.x * blockDim.x) {
        const size_t row = i / vecs_per_row;
        const int c = (int)(i - row * vecs_per_row) * 8;
        const uint4 ar = *(const uint4*)(a + row * cols + c);
        const float s = 1.0f / (1.0f + expf(-ld(g + row * g_ld + g_off + c / group)));
        const uint32_t aw[4] = {ar.x, ar.y, ar.z, ar.w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            o[j] = pack_bf16x2(__uint_as_float(aw[j] << 16) * s, __uint_as_float(aw[j] & 0xffff0000u) * s);
        *(uint4*)(a + row * cols + c) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// group: columns that share one gate value (1: a value a column; a head's width: a value a head)
extern "C" int ia_sigmoid_gate(void* a, const void* g, int rows, int cols, int g_ld, int g_off, int group, int dtype,
                               hipStream_t stream) {
    IA_CHECK(rows >= 0 && cols > 0 && group >= 1 && cols % group == 0 && g_off >= 0 && g_off + cols / group <= g_ld,
             "sigmoid_gate: rows=%d cols=%d pitch=%d offset=%d group=%d", rows, cols, g_ld, g_off, group);
    if (rows == 0) return 0;
    const size_t total = (size_t)rows * cols;
    const int block = 256;
    if (group == 1 && dtype == IA_BF16 && cols % 8 == 0 && g_ld % 8 == 0 && g_off % 8 == 0 && ((((uintptr_t)a) | ((uintptr_t)g)) & 15) == 0) {
        const size_t vecs = total / 8;
        const size_t want = (vecs + block - 1) / block;
        sigmoid_gate_bf16_vec_kernel<<<(unsigned)(want < 65535 * 8 ? want : 65535 * 8), block, 0, stream>>>(
            (bf16_t*)a, (const bf16_t*)g, cols, g_ld, g_off, vecs);
        IA_LAUNCH_CHECK("sigmoid_gate");
        return 0;
    }
    if (group % 8 == 0 && dtype == IA_BF16 && (((uintptr_t)a) & 15) == 0) {
        const size_t vecs = total / 8;
        const size_t want = (vecs + block - 1) / block;
        sigmoid_gate_group_bf16_vec_kernel<<<(unsigned)(want < 65535 * 8 ? want : 65535 * 8), block, 0, stream>>>(
            (bf16_t*)a, (const bf16_t*)g, cols, g_ld, g_off, group, vecs);
        IA_LAUNCH_CHECK("sigmoid_gate");
        return 0;
    }
    const size_t want = (total + block - 1) / block;
    const int grid = (int)(want < 65535 ? want : 65535);
    if (dtype == IA_F32)
        sigmoid_gate_kernel<float><<<grid, block, 0, stream>>>((float*)a, (const float*)g, cols, g_ld, g_off, group, total);
    else if (dtype == IA_BF16)
        sigmoid_gate_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)a, (const bf16_t*)g, cols, g_ld, g_off, group, total);
    else
        IA_CHECK(false, "sigmoid_gate: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("sigmoid_gate");
    return 0;
}

// ---- rows of [gate | up] -> g' * sigmoid(slope g') * (u' + 1), g' = min(gate, limit), u' = clamp(up, -limit, limit) ------
__device__ __forceinline__ float clamped_gate(float g, float u, float limit, float slope) {
    const float gv = fminf(g, limit), uv = fminf(fmaxf(u, -limit), limit);
    return gv / (1.0f + expf(-slope * gv)) * (uv + 1.0f);
}

template <typename T>
__global__ void clamped_gate_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, int inter, size_t total, float limit,
                                        float slope) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t row = i / inter;
        const int c = (int)(i - row * inter);
        st(out + i, clamped_gate(ld(gu + row * 2 * inter + c), ld(gu + row * 2 * inter + inter + c), limit, slope));
    }
}

__global__ void clamped_gate_mul_bf16_vec_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ gu, int inter,
                                                 size_t total_vecs, float limit, float slope) {
    const int vecs_per_row = inter / 8;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total_vecs; i += (size_t)gridDim.x * blockDim.x) {
        const size_t row = i / vecs_per_row;
        const int c = (int)(i - row * vecs_per_row) * 8;
        const uint4 gr = *(const uint4*)(gu + row * 2 * inter + c);
        const uint4 ur = *(const uint4*)(gu + row * 2 * inter + inter + c);
        const uint32_t gw[4] = {gr.x, gr.y, gr.z, gr.w}, uw[4] = {ur.x, ur.y, ur.z, ur.w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
            const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
            o[j] = pack_bf16x2(clamped_gate(g0, u0, limit, slope), clamped_gate(g1, u1, limit, slope));
        }
        *(uint4*)(out + row * inter + c) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

extern "C" int ia_clamped_gate_mul(void* out, const void* gu, int rows, int inter, float limit, float slope, int dtype,
                                   hipStream_t stream) {
    IA_CHECK(rows >= 0 && inter > 0 && limit > 0.f, "clamped_gate_mul: bad sizes rows=%d inter=%d limit=%g", rows, inter, (double)limit);
    if (rows == 0) return 0;
    const size_t total = (size_t)rows * inter;
    const int block = 256;
    if (dtype == IA_BF16 && inter % 8 == 0 && ((((uintptr_t)out) | ((uintptr_t)gu)) & 15) == 0) {
        const size_t vecs = total / 8;
        const size_t want = (vecs + block - 1) / block;
        clamped_gate_mul_bf16_vec_kernel<<<(unsigned)(want < 65535 * 8 ? want : 65535 * 8), block, 0, stream>>>(
            (bf16_t*)out, (const bf16_t*)gu, inter, vecs, limit, slope);
        IA_LAUNCH_CHECK("clamped_gate_mul");
        return 0;
    }
    const size_t want = (total + block - 1) / block;
    const int grid = (int)(want < 65535 ? want : 65535);
    if (dtype == IA_F32)
        clamped_gate_mul_kernel<float><<<grid, block, 0, stream>>>((float*)out, (const float*)gu, inter, total, limit, slope);
    else if (dtype == IA_BF16)
        clamped_gate_mul_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, inter, total, limit, slope);
    else
        IA_CHECK(false, "clamped_gate_mul: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("clamped_gate_mul");
    return 0;
}

// ---- x *= factor over 32-bit values in place ---------------------------------------------------------------------------
__global__ void scale_kernel(float* __restrict__ x, size_t n, float factor) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) x[i] *= factor;
}

extern "C" int ia_scale(float* x, long long n, float factor, hipStream_t stream) {
    IA_CHECK(n >= 0, "scale: n=%lld", n);
    if (n == 0) return 0;
    const size_t want = ((size_t)n + 255) / 256;
    scale_kernel<<<(unsigned)(want < 65535 ? want : 65535), 256, 0, stream>>>(x, (size_t)n, factor);
    IA_LAUNCH_CHECK("scale");
    return 0;
}
