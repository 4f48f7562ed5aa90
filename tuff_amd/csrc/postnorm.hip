// Kernels of layers that norm a sublayer's output before it joins the residual stream, all in float32.
//
// tuff_post_norm_add, a workgroup a token:
//     x <- x + mult * y / sqrt(mean(y^2) + eps) * w  [+ extra]        (y is then cleared, if asked, or set to a row
//                                                                      y_next: the bias of the product that adds into y next)
//     h  = x / sqrt(mean(x^2) + eps_next) * w_next                     (if asked: the next sublayer's input)
// One launch where a norm, a residual sum, another sum and the next norm would be four.  Without y only the
// sum with `extra` and the next norm run.  The weights come in as float32 with any offset already added.
//
// tuff_normed_mean2, a workgroup a token:
//     out <- out + coef * (a / sqrt(mean(a^2) + eps) * wa + b / sqrt(mean(b^2) + eps) * wb)
// for a mixer made of two mixers side by side whose outputs are each normed over the width.
//
// tuff_scale_add_layer_norm, a workgroup a token, for layers that scale a sublayer's output per channel:
//     x <- x + ls * y                                                   (y is then cleared, if asked)
//     h  = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * w_next   (if asked: the next sublayer's input)
// a layer norm with a weight and no bias, the variance taken from the deviations themselves.  Without y the norm
// alone runs, then optionally over chosen rows of x only (the rows whose logits are wanted).
//
// Every row's sums run over the row in one fixed order (a thread's elements in ascending order, the
// butterfly of a wave, the waves in order), so a row's result does not depend on what else is in the step.
#include "common.h"
#include <math.h>

namespace {
constexpr int PN_THREADS = 256;
constexpr int PN_WAVES = PN_THREADS / WAVE;

template <typename T>
__global__ __launch_bounds__(PN_THREADS) void post_norm_add_kernel(
    float* __restrict__ x, float* __restrict__ y, const float* __restrict__ w, float eps, float mult,
    const float* __restrict__ extra, const float* __restrict__ w_next, float eps_next, T* __restrict__ h_out,
    int d, int clear_y, const float* __restrict__ y_next) {
    __shared__ float scratch[PN_WAVES];
    const long long row = (long long)blockIdx.x * d;
    float* xr = x + row;
    float inv = 0.f;
    if (y) {
        const float* yr = y + row;
        float ss = 0.f;
        for (int c = threadIdx.x; c < d; c += PN_THREADS) ss = fmaf(yr[c], yr[c], ss);
        ss = block_sum<PN_WAVES>(ss, scratch);
        inv = mult / sqrtf(ss / (float)d + eps);
    }
    float ss2 = 0.f;
    for (int c = threadIdx.x; c < d; c += PN_THREADS) {
        float v = xr[c];
        if (y) {
            v = fmaf(y[row + c] * inv, w[c], v);
            if (clear_y) y[row + c] = y_next ? y_next[c] : 0.f;
        }
        if (extra) v += extra[row + c];
        if (y || extra) xr[c] = v;
        ss2 = fmaf(v, v, ss2);
    }
    if (!h_out) return;
    ss2 = block_sum<PN_WAVES>(ss2, scratch);
    const float inv2 = 1.0f / sqrtf(ss2 / (float)d + eps_next);
    // (a thread reads back the elements it wrote itself)
    for (int c = threadIdx.x; c < d; c += PN_THREADS) h_out[row + c] = from_f32<T>(xr[c] * inv2 * w_next[c]);
}

// The same for rows of at most PN_THREADS * EPT elements: a thread keeps its elements in registers, and everything a
// row needs is loaded before the first sum, so the launch waits for memory once.  The sums run in the order of the
// kernel above (a thread's elements in ascending order): the same bits.
template <typename T, int EPT>
__global__ __launch_bounds__(PN_THREADS) void post_norm_add_regs_kernel(
    float* __restrict__ x, float* __restrict__ y, const float* __restrict__ w, float eps, float mult,
    const float* __restrict__ extra, const float* __restrict__ w_next, float eps_next, T* __restrict__ h_out,
    int d, int clear_y, const float* __restrict__ y_next) {
    __shared__ float scratch[PN_WAVES];
    const long long row = (long long)blockIdx.x * d;
    float xv[EPT], yv[EPT], wv[EPT], ev[EPT], nv[EPT];
#pragma unroll
    for (int k = 0; k < EPT; ++k) {
        const int c = threadIdx.x + k * PN_THREADS;
        const bool in = c < d;
        xv[k] = in ? x[row + c] : 0.f;
        yv[k] = (in && y) ? y[row + c] : 0.f;
        wv[k] = (in && y) ? w[c] : 0.f;
        ev[k] = (in && extra) ? extra[row + c] : 0.f;
        nv[k] = (in && h_out) ? w_next[c] : 0.f;
    }
    float inv = 0.f;
    if (y) {
        float ss = 0.f;
#pragma unroll
        for (int k = 0; k < EPT; ++k)
            if (threadIdx.x + k * PN_THREADS < d) ss = fmaf(yv[k], yv[k], ss);
        ss = block_sum<PN_WAVES>(ss, scratch);
        inv = mult / sqrtf(ss / (float)d + eps);
    }
    float ss2 = 0.f;
#pragma unroll
    for (int k = 0; k < EPT; ++k) {
        const int c = threadIdx.x + k * PN_THREADS;
        if (c >= d) continue;
        float v = xv[k];
        if (y) {
            v = fmaf(yv[k] * inv, wv[k], v);
            if (clear_y) y[row + c] = y_next ? y_next[c] : 0.f;
        }
        if (extra) v += ev[k];
        if (y || extra) x[row + c] = v;
        xv[k] = v;
        ss2 = fmaf(v, v, ss2);
    }
    if (!h_out) return;
    ss2 = block_sum<PN_WAVES>(ss2, scratch);
    const float inv2 = 1.0f / sqrtf(ss2 / (float)d + eps_next);
#pragma unroll
    for (int k = 0; k < EPT; ++k) {
        const int c = threadIdx.x + k * PN_THREADS;
        if (c < d) h_out[row + c] = from_f32<T>(xv[k] * inv2 * nv[k]);
    }
}

__global__ __launch_bounds__(PN_THREADS) void normed_mean2_kernel(
    const float* __restrict__ a, const float* __restrict__ wa, const float* __restrict__ b, const float* __restrict__ wb,
    float eps, float coef, float* __restrict__ out, int d) {
    __shared__ float scratch[PN_WAVES];
    const long long row = (long long)blockIdx.x * d;
    float sa = 0.f, sb = 0.f;
    for (int c = threadIdx.x; c < d; c += PN_THREADS) {
        sa = fmaf(a[row + c], a[row + c], sa);
        sb = fmaf(b[row + c], b[row + c], sb);
    }
    sa = block_sum<PN_WAVES>(sa, scratch);
    sb = block_sum<PN_WAVES>(sb, scratch);
    const float ia = 1.0f / sqrtf(sa / (float)d + eps), ib = 1.0f / sqrtf(sb / (float)d + eps);
    for (int c = threadIdx.x; c < d; c += PN_THREADS)
        out[row + c] += coef * (a[row + c] * ia * wa[c] + b[row + c] * ib * wb[c]);
}

// EPT > 0: rows of at most PN_THREADS * EPT elements stay in registers between the sums; EPT 0: any width, the row
// read again from x for every pass (a thread reads back what it wrote itself).  The sums run in the same order.
template <typename T, int EPT>
__global__ __launch_bounds__(PN_THREADS) void scale_add_layer_norm_kernel(
    float* __restrict__ x, float* __restrict__ y, const float* __restrict__ ls, const float* __restrict__ w_next, float eps,
    T* __restrict__ h_out, const int* __restrict__ rows, int d, int clear_y) {
    __shared__ float scratch[PN_WAVES];
    const long long src = (long long)(rows ? rows[blockIdx.x] : (int)blockIdx.x) * d;
    const long long dst = (long long)blockIdx.x * d;
    constexpr int N = EPT > 0 ? EPT : 1;
    float xv[N];
    float sum = 0.f;
    float nv[N];                                       // the next norm's weight: asked for with everything else, before the first sum
    if (EPT > 0) {
        float yv[N], lv[N];
#pragma unroll
        for (int k = 0; k < N; ++k) {
            const int c = threadIdx.x + k * PN_THREADS;
            const bool in = c < d;
            xv[k] = in ? x[src + c] : 0.f;
            yv[k] = (in && y) ? y[src + c] : 0.f;
            lv[k] = (in && y) ? ls[c] : 0.f;
            nv[k] = (in && h_out) ? w_next[c] : 0.f;
        }
#pragma unroll
        for (int k = 0; k < N; ++k) {
            const int c = threadIdx.x + k * PN_THREADS;
            if (c >= d) continue;
            if (y) {
                xv[k] = fmaf(lv[k], yv[k], xv[k]);
                x[src + c] = xv[k];
                if (clear_y) y[src + c] = 0.f;
            }
            sum += xv[k];
        }
    } else {
        for (int c = threadIdx.x; c < d; c += PN_THREADS) {
            float v = x[src + c];
            if (y) {
                v = fmaf(ls[c], y[src + c], v);
                x[src + c] = v;
                if (clear_y) y[src + c] = 0.f;
            }
            sum += v;
        }
    }
    if (!h_out) return;
    const float mean = block_sum<PN_WAVES>(sum, scratch) / (float)d;
    float ss = 0.f;
    if (EPT > 0) {
#pragma unroll
        for (int k = 0; k < N; ++k)
            if (threadIdx.x + k * PN_THREADS < d) { const float dv = xv[k] - mean; ss = fmaf(dv, dv, ss); }
    } else {
        for (int c = threadIdx.x; c < d; c += PN_THREADS) { const float dv = x[src + c] - mean; ss = fmaf(dv, dv, ss); }
    }
    __syncthreads();                                   // (the scratch of the first sum is read by all before it is used again)
    ss = block_sum<PN_WAVES>(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    if (EPT > 0) {
#pragma unroll
        for (int k = 0; k < N; ++k) {
            const int c = threadIdx.x + k * PN_THREADS;
            if (c < d) h_out[dst + c] = from_f32<T>((xv[k] - mean) * inv * nv[k]);
        }
    } else {
        for (int c = threadIdx.x; c < d; c += PN_THREADS) h_out[dst + c] = from_f32<T>((x[src + c] - mean) * inv * w_next[c]);
    }
}
}  // namespace

// x float32 [T][d] in place; y float32 [T][d] with ls float32 [d], or both null; w_next float32 [d] and h_out [n_rows][d]
// of type out_dt, or both null; rows int32 [n_rows] or null (only without y): the rows of x that are normed, in
// this order; without it n_rows = T and row i is normed into row i.
TUFF_EXPORT int tuff_scale_add_layer_norm(float* x, float* y, const float* ls, const float* w_next, float eps, void* h_out,
                                          int out_dt, const int* rows, int n_rows, int d, int clear_y, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (d <= 0 || ((y == nullptr) != (ls == nullptr)) || ((w_next == nullptr) != (h_out == nullptr)) || (rows && y)) return -2;
    dim3 grid(n_rows), block(PN_THREADS);
#define LAUNCH(E, T) hipLaunchKernelGGL((scale_add_layer_norm_kernel<T, E>), grid, block, 0, stream, x, y, ls, w_next, eps, (T*)h_out, rows, d, clear_y)
    if (d <= PN_THREADS * 4) { if (out_dt == DT_F32) LAUNCH(4, float); else LAUNCH(4, bf16_t); }
    else if (d <= PN_THREADS * 16) { if (out_dt == DT_F32) LAUNCH(16, float); else LAUNCH(16, bf16_t); }
    else { if (out_dt == DT_F32) LAUNCH(0, float); else LAUNCH(0, bf16_t); }
#undef LAUNCH
    return launch_status();
}

// x float32 [T][d] in place; y float32 [T][d] or null; w float32 [d] (with y); extra float32 [T][d] or null;
// w_next float32 [d] and h_out [T][d] of type out_dt, or both null; y_next float32 [d] or null (with clear_y).
TUFF_EXPORT int tuff_post_norm_add(float* x, float* y, const float* w, float eps, float mult, const float* extra,
                                   const float* w_next, float eps_next, void* h_out, int out_dt, int n_tokens, int d,
                                   int clear_y, const float* y_next, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (d <= 0 || (y && !w) || ((w_next == nullptr) != (h_out == nullptr))) return -2;
    dim3 grid(n_tokens), block(PN_THREADS);
#define LAUNCH(KERN, T) hipLaunchKernelGGL(KERN, grid, block, 0, stream, x, y, w, eps, mult, extra, w_next, eps_next, (T*)h_out, d, clear_y, y_next)
    if (d <= PN_THREADS * 8) {
        if (out_dt == DT_F32) LAUNCH((post_norm_add_regs_kernel<float, 8>), float); else LAUNCH((post_norm_add_regs_kernel<bf16_t, 8>), bf16_t);
    } else if (d <= PN_THREADS * 32) {
        if (out_dt == DT_F32) LAUNCH((post_norm_add_regs_kernel<float, 32>), float); else LAUNCH((post_norm_add_regs_kernel<bf16_t, 32>), bf16_t);
    } else {
        if (out_dt == DT_F32) LAUNCH(post_norm_add_kernel<float>, float); else LAUNCH(post_norm_add_kernel<bf16_t>, bf16_t);
    }
#undef LAUNCH
    return launch_status();
}

TUFF_EXPORT int tuff_normed_mean2(const float* a, const float* wa, const float* b, const float* wb, float eps, float coef,
                                  float* out, int n_tokens, int d, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (d <= 0) return -2;
    hipLaunchKernelGGL(normed_mean2_kernel, dim3(n_tokens), dim3(PN_THREADS), 0, stream, a, wa, b, wb, eps, coef, out, d);
    return launch_status();
}
