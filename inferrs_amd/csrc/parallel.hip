// A layer whose sub-layers all read ONE normed copy of a 32-bit residual stream and whose outputs are added together:
//     x <- x + y1 (+ y2) (+ sum_k [w_k] r_k) (+ s y3)          the sub-layers' outputs, every one optional
//     x <- x + rmsnorm(t) * w_t                                  (optional) a row that enters behind the sum, normed
//     h  = norm(x)                                               (optional) what the next layer's sub-layers read
// ONE kernel does any of these three in that order: a block owns a row, the sum stays in shared memory between them,
// every statistic is 32-bit.  y1, y2, y3 may each be a product still split along its k ([splits, n, W], 32-bit); r_k
// are the rows of routed experts [n, top, W] (32-bit) with weights w_k or, without, added as they are; s is one
// 32-bit factor a row.  The norm at the end is a layer norm, (x - mean) / sqrt(var + eps) * w + b with the variance the
// mean of the squared deviations from the mean, or, with `center` 0, an RMS norm (b may be null).  The new x can be
// written once more in the products' precision (`xr`).  With `rows` the kernel reads the named rows only, adds nothing
// and leaves the stream alone (the model's end: the wanted rows through the final norm).
//
// Beside it: act(g) * e for rows g and a slice of wider rows e (a token's own input, gated).
#include "api.h"
#include "common.h"

#define PL_MAX_TOP 16

template <typename T>
__device__ __forceinline__ float pl_sum_splits(const T* p, int splits, long long stride) {
    float t = ld(p);
    for (int s = 1; s < splits; ++s) t += ld(p + s * stride);
    return t;
}

template <typename TY, typename TH>
__global__ __launch_bounds__(1024) void parallel_step_kernel(
    float* __restrict__ x, const TY* __restrict__ y1, const TY* __restrict__ y2, const TY* __restrict__ y3, int y1_splits,
    int y2_splits, int y3_splits, long long split_stride, const float* __restrict__ y3_scale,
    const float* __restrict__ routed, const float* __restrict__ routed_w, int top, const TY* __restrict__ enter,
    const float* __restrict__ enter_w, float enter_eps, TH* __restrict__ xr, const float* __restrict__ norm_w,
    const float* __restrict__ norm_b, float norm_eps, int center, TH* __restrict__ h, const int* __restrict__ rows, int W) {
    extern __shared__ float pl_row[];            // [W]
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int row = rows != nullptr ? rows[r] : r;
    float* xrow = x + (long long)row * W;
    const long long at = (long long)row * W;
    const float s3 = y3 != nullptr && y3_scale != nullptr ? y3_scale[row] : 1.0f;
    float wk[PL_MAX_TOP];
#pragma unroll
    for (int k = 0; k < PL_MAX_TOP; ++k) wk[k] = routed != nullptr && routed_w != nullptr && k < top ? routed_w[(long long)row * top + k] : 1.0f;
    float sq = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float v = xrow[c];
        if (y1 != nullptr) v += pl_sum_splits(y1 + at + c, y1_splits, split_stride);
        if (y2 != nullptr) v += pl_sum_splits(y2 + at + c, y2_splits, split_stride);
        if (routed != nullptr) {
#pragma unroll
            for (int k = 0; k < PL_MAX_TOP; ++k)
                if (k < top) v = fmaf(wk[k], routed[((long long)row * top + k) * W + c], v);
        }
        if (y3 != nullptr) v = fmaf(s3, pl_sum_splits(y3 + at + c, y3_splits, split_stride), v);
        pl_row[c] = v;
        if (enter != nullptr) {
            const float e = ld(enter + at + c);
            sq = fmaf(e, e, sq);
        }
    }
    if (enter != nullptr) {
        const float rs = 1.0f / sqrtf(block_sum(sq, scratch) / (float)W + enter_eps);
        for (int c = threadIdx.x; c < W; c += blockDim.x) pl_row[c] += ld(enter + at + c) * rs * enter_w[c];
    }
    // (a thread reads back the features it wrote: no barrier is needed up to here)
    if (rows == nullptr) {
        for (int c = threadIdx.x; c < W; c += blockDim.x) {
            const float v = pl_row[c];
            xrow[c] = v;
            if (xr != nullptr) st(xr + at + c, v);
        }
    }
    if (h == nullptr) return;
    float mean = 0.f;
    if (center) {
        float sum = 0.f;
        for (int c = threadIdx.x; c < W; c += blockDim.x) sum += pl_row[c];
        mean = block_sum(sum, scratch) / (float)W;
    }
    float dev = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float d = pl_row[c] - mean;
        dev = fmaf(d, d, dev);
    }
    const float rs = 1.0f / sqrtf(block_sum(dev, scratch) / (float)W + norm_eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float v = (pl_row[c] - mean) * rs * norm_w[c];
        if (norm_b != nullptr) v += norm_b[c];
        st(h + (long long)r * W + c, v);
    }
}

// The same for widths in steps of 8 up to 8 * PL_VEC_ITERS * the block's threads: a thread owns eight neighbouring features
// a round (16- and 32-byte accesses), the row's sum stays in its registers between the steps, and nothing goes through
// shared memory but the statistics.  The arithmetic of a feature is that of the kernel above.
#define PL_VEC_ITERS 4

__device__ __forceinline__ void pl_load8(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void pl_load8(const bf16_t* p, float (&v)[8]) {
    const uint4 a = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}
__device__ __forceinline__ void pl_store8(float* p, const float (&v)[8]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void pl_store8(bf16_t* p, const float (&v)[8]) {
    *reinterpret_cast<uint4*>(p) = make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]),
                                              pack_bf16x2(v[6], v[7]));
}
template <typename T>
__device__ __forceinline__ void pl_load8_splits(const T* p, int splits, long long stride, float (&t)[8]) {
    pl_load8(p, t);
    for (int s = 1; s < splits; ++s) {
        float u[8];
        pl_load8(p + s * stride, u);
#pragma unroll
        for (int i = 0; i < 8; ++i) t[i] += u[i];
    }
}

template <typename TY, typename TH>
__global__ __launch_bounds__(1024) void parallel_step_vec_kernel(
    float* __restrict__ x, const TY* __restrict__ y1, const TY* __restrict__ y2, const TY* __restrict__ y3, int y1_splits,
    int y2_splits, int y3_splits, long long split_stride, const float* __restrict__ y3_scale,
    const float* __restrict__ routed, const float* __restrict__ routed_w, int top, const TY* __restrict__ enter,
    const float* __restrict__ enter_w, float enter_eps, TH* __restrict__ xr, const float* __restrict__ norm_w,
    const float* __restrict__ norm_b, float norm_eps, int center, TH* __restrict__ h, const int* __restrict__ rows, int W) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int row = rows != nullptr ? rows[r] : r;
    const long long at = (long long)row * W;
    float* xrow = x + at;
    const float s3 = y3 != nullptr && y3_scale != nullptr ? y3_scale[row] : 1.0f;
    float wk[PL_MAX_TOP];
#pragma unroll
    for (int k = 0; k < PL_MAX_TOP; ++k) wk[k] = routed != nullptr && routed_w != nullptr && k < top ? routed_w[(long long)row * top + k] : 1.0f;
    float v[PL_VEC_ITERS][8], e[PL_VEC_ITERS][8];
    float sq = 0.f;
#pragma unroll
    for (int it = 0; it < PL_VEC_ITERS; ++it) {
        const int c = (it * blockDim.x + threadIdx.x) * 8;
        if (c >= W) continue;
        float t[8];
        pl_load8(xrow + c, v[it]);
        if (y1 != nullptr) {
            pl_load8_splits(y1 + at + c, y1_splits, split_stride, t);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[it][i] += t[i];
        }
        if (y2 != nullptr) {
            pl_load8_splits(y2 + at + c, y2_splits, split_stride, t);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[it][i] += t[i];
        }
        if (routed != nullptr) {
#pragma unroll
            for (int k = 0; k < PL_MAX_TOP; ++k) {
                if (k >= top) break;
                pl_load8(routed + ((long long)row * top + k) * W + c, t);
#pragma unroll
                for (int i = 0; i < 8; ++i) v[it][i] = fmaf(wk[k], t[i], v[it][i]);
            }
        }
        if (y3 != nullptr) {
            pl_load8_splits(y3 + at + c, y3_splits, split_stride, t);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[it][i] = fmaf(s3, t[i], v[it][i]);
        }
        if (enter != nullptr) {
            pl_load8(enter + at + c, e[it]);
#pragma unroll
            for (int i = 0; i < 8; ++i) sq = fmaf(e[it][i], e[it][i], sq);
        }
    }
    if (enter != nullptr) {
        const float rs = 1.0f / sqrtf(block_sum(sq, scratch) / (float)W + enter_eps);
#pragma unroll
        for (int it = 0; it < PL_VEC_ITERS; ++it) {
            const int c = (it * blockDim.x + threadIdx.x) * 8;
            if (c >= W) continue;
            float wv[8];
            pl_load8(enter_w + c, wv);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[it][i] += e[it][i] * rs * wv[i];
        }
    }
    if (rows == nullptr) {
#pragma unroll
        for (int it = 0; it < PL_VEC_ITERS; ++it) {
            const int c = (it * blockDim.x + threadIdx.x) * 8;
            if (c >= W) continue;
            pl_store8(xrow + c, v[it]);
            if (xr != nullptr) pl_store8(xr + at + c, v[it]);
        }
    }
    if (h == nullptr) return;
    float mean = 0.f;
    if (center) {
        float sum = 0.f;
#pragma unroll
        for (int it = 0; it < PL_VEC_ITERS; ++it) {
            const int c = (it * blockDim.x + threadIdx.x) * 8;
            if (c >= W) continue;
#pragma unroll
            for (int i = 0; i < 8; ++i) sum += v[it][i];
        }
        mean = block_sum(sum, scratch) / (float)W;
    }
    float dev = 0.f;
#pragma unroll
    for (int it = 0; it < PL_VEC_ITERS; ++it) {
        const int c = (it * blockDim.x + threadIdx.x) * 8;
        if (c >= W) continue;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float d = v[it][i] - mean;
            dev = fmaf(d, d, dev);
        }
    }
    const float rs = 1.0f / sqrtf(block_sum(dev, scratch) / (float)W + norm_eps);
#pragma unroll
    for (int it = 0; it < PL_VEC_ITERS; ++it) {
        const int c = (it * blockDim.x + threadIdx.x) * 8;
        if (c >= W) continue;
        float wv[8], o[8];
        pl_load8(norm_w + c, wv);
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = (v[it][i] - mean) * rs * wv[i];
        if (norm_b != nullptr) {
            pl_load8(norm_b + c, wv);
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] += wv[i];
        }
        pl_store8(h + (long long)r * W + c, o);
    }
}

// y_dtype: precision of y1, y2, y3 and enter; h_dtype: of xr and h.  0 float32, 1 bfloat16.  Outputs in more than one split
// are 32-bit and cover every row.
extern "C" int ia_parallel_step(float* x, const void* y1, const void* y2, const void* y3, int y1_splits, int y2_splits,
                                int y3_splits, const float* y3_scale, const float* routed, const float* routed_w, int top,
                                const void* enter, const float* enter_w, float enter_eps, void* xr, const float* norm_w,
                                const float* norm_b, float norm_eps, int center, void* h, const int* rows, int n, int W,
                                int y_dtype, int h_dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && W > 0 && x != nullptr, "parallel_step: n=%d width=%d, and the stream", n, W);
    IA_CHECK((size_t)W * sizeof(float) <= 60 * 1024, "parallel_step: width %d does not fit shared memory", W);
    IA_CHECK(routed == nullptr || (top >= 1 && top <= PL_MAX_TOP), "parallel_step: up to %d routed rows a row (top=%d)", PL_MAX_TOP, top);
    IA_CHECK(enter == nullptr || enter_w != nullptr, "parallel_step: a row that enters comes with its norm's weight");
    IA_CHECK(h == nullptr || norm_w != nullptr, "parallel_step: normed rows come with the norm's weight");
    IA_CHECK(rows == nullptr || (h != nullptr && y1 == nullptr && y2 == nullptr && y3 == nullptr && routed == nullptr &&
                                 enter == nullptr && xr == nullptr),
             "parallel_step: a row list leaves the stream alone: normed rows out, nothing added");
    IA_CHECK(y1_splits >= 1 && y2_splits >= 1 && y3_splits >= 1 &&
                 ((y1_splits == 1 && y2_splits == 1 && y3_splits == 1) || y_dtype == IA_F32),
             "parallel_step: outputs in %d, %d and %d splits are 32-bit", y1_splits, y2_splits, y3_splits);
    if (n == 0) return 0;
    const long long split_stride = (long long)n * W;
    const uintptr_t ptrs = (uintptr_t)x | (uintptr_t)y1 | (uintptr_t)y2 | (uintptr_t)y3 | (uintptr_t)routed | (uintptr_t)enter |
                           (uintptr_t)enter_w | (uintptr_t)xr | (uintptr_t)norm_w | (uintptr_t)norm_b | (uintptr_t)h;
    if (W % 8 == 0 && (ptrs & 15) == 0 && W <= 8 * PL_VEC_ITERS * 1024) {
        // as many threads as the row has pieces of eight, in whole waves, a round or more each
        int vthreads = (W / 8 + 63) / 64 * 64;
        if (vthreads > 256) vthreads = (W / 8 + 2 * 64 - 1) / (2 * 64) * 64;          // two rounds a thread
        if (vthreads > 512) vthreads = (W / 8 + PL_VEC_ITERS * 64 - 1) / (PL_VEC_ITERS * 64) * 64;
#define IA_LAUNCH_VEC(TY, TH)                                                                                            \
    parallel_step_vec_kernel<TY, TH><<<n, vthreads, 0, stream>>>(x, (const TY*)y1, (const TY*)y2, (const TY*)y3, y1_splits, \
                                                                 y2_splits, y3_splits, split_stride, y3_scale, routed,      \
                                                                 routed_w, top, (const TY*)enter, enter_w, enter_eps,       \
                                                                 (TH*)xr, norm_w, norm_b, norm_eps, center, (TH*)h, rows, W)
        if (y_dtype == IA_F32 && h_dtype == IA_F32) { IA_LAUNCH_VEC(float, float); }
        else if (y_dtype == IA_F32) { IA_LAUNCH_VEC(float, bf16_t); }
        else if (h_dtype == IA_F32) { IA_LAUNCH_VEC(bf16_t, float); }
        else { IA_LAUNCH_VEC(bf16_t, bf16_t); }
#undef IA_LAUNCH_VEC
        IA_LAUNCH_CHECK("parallel_step");
        return 0;
    }
    const int threads = W >= 4096 ? 1024 : W >= 1024 ? 512 : W >= 512 ? 256 : 128;
    const size_t shm = (size_t)W * sizeof(float);
#define IA_LAUNCH(TY, TH)                                                                                              \
    parallel_step_kernel<TY, TH><<<n, threads, shm, stream>>>(x, (const TY*)y1, (const TY*)y2, (const TY*)y3, y1_splits,  \
                                                              y2_splits, y3_splits, split_stride, y3_scale, routed,      \
                                                              routed_w, top, (const TY*)enter, enter_w, enter_eps,       \
                                                              (TH*)xr, norm_w, norm_b, norm_eps, center, (TH*)h, rows, W)
    if (y_dtype == IA_F32 && h_dtype == IA_F32) { IA_LAUNCH(float, float); }
    else if (y_dtype == IA_F32) { IA_LAUNCH(float, bf16_t); }
    else if (h_dtype == IA_F32) { IA_LAUNCH(bf16_t, float); }
    else { IA_LAUNCH(bf16_t, bf16_t); }
#undef IA_LAUNCH
    IA_LAUNCH_CHECK("parallel_step");
    return 0;
}

// ---- out[t][c] = act(g[t][c]) * e[t][e_off + c] --------------------------------------------------------------------------
template <typename T>
__global__ void gate_rows_kernel(T* __restrict__ out, const T* __restrict__ g, const T* __restrict__ e, int cols,
                                 long long e_ld, int e_off, int act, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t row = i / cols;
        const int c = (int)(i - row * cols);
        st(out + i, gate_act(ld(g + i), act) * ld(e + row * e_ld + e_off + c));
    }
}

// act: 1 SiLU, 2 GELU in its tanh form (common.h).  g and out [rows, cols] contiguous; e rows of pitch e_ld.
extern "C" int ia_gate_rows(void* out, const void* g, const void* e, int rows, int cols, long long e_ld, int e_off, int act,
                            int dtype, hipStream_t stream) {
    IA_CHECK(rows >= 0 && cols > 0 && e_off >= 0 && e_off + cols <= e_ld, "gate_rows: rows=%d cols=%d pitch=%lld offset=%d", rows,
             cols, e_ld, e_off);
    IA_CHECK(act >= IA_ACT_SILU && act <= IA_ACT_LAST, "gate_rows: unknown activation %d", act);
    if (rows == 0) return 0;
    const size_t total = (size_t)rows * cols;
    const int block = 256;
    const size_t want = (total + block - 1) / block;
    const int grid = (int)(want < 65535 ? want : 65535);
    if (dtype == IA_F32)
        gate_rows_kernel<float><<<grid, block, 0, stream>>>((float*)out, (const float*)g, (const float*)e, cols, e_ld, e_off, act, total);
    else if (dtype == IA_BF16)
        gate_rows_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)out, (const bf16_t*)g, (const bf16_t*)e, cols, e_ld, e_off, act, total);
    else
        IA_CHECK(false, "gate_rows: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("gate_rows");
    return 0;
}
