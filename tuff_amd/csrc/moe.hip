// Mixture of experts: the choice of experts per token and the chosen experts' two products.
//
// Routing: from router logits z [T][E] (float32) the `top` largest are chosen per token (the lower
// index wins a tie); the weight of a choice is f(z): 0 sigmoid (each score on its own, not
// renormalised), 1 softmax over the chosen.  Everything here is float32.
//
// Experts: y = W_down act(W_up x) with x the token's input, multiplied by the choice's weight before
// (scale_input) or y after; act: 0 relu squared, 1 silu, 2 gelu (tanh form).  Gated experts have two first
// matrices: y = W_down glu(W_gate x, W_up x) with glu(g, u) = act(g) u for the three above, or, act 3, the
// clamped form g' sigmoid(alpha g') (u' + 1) with g' = min(g, limit), u' = clamp(u, -limit, limit).
// The router may have a bias: z = W h + b.  A limited choice (sigmoid weights): the choice runs on
// c = sigmoid(z) + correction instead of z, and only inside the `keep` groups of neighbouring experts (of `groups`
// equal ones) whose two largest c have the largest sum; the weights are the chosen experts' sigmoid(z), without the
// correction, times a constant.  A (token, choice) pair is a
// row of the work arrays; the rows of a token are added into the residual stream in the order of
// its choices, so the sum does not depend on what else is in the step.
#include "common.h"
#include <math.h>

namespace {
__device__ __forceinline__ float act_fn(float z, int act) {
    if (act == 0) { const float r = fmaxf(z, 0.f); return r * r; }
    if (act == 1) return z / (1.0f + expf(-z));
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// What a gated expert makes of its two products (see the head of the file).
__device__ __forceinline__ float glu_fn(float g, float u, int act, float limit, float alpha) {
    if (act != 3) return act_fn(g, act) * u;
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
}

// The `top` largest of row[0..E-1] in the order (value descending, index ascending) and their weights.
__device__ void choose(const float* row, int* ids, float* wts, long long t, int E, int top, int weight_fn) {
    float last = INFINITY;
    int last_id = -1;
    float zmax = 0.f, den = 0.f;
    for (int s = 0; s < top; ++s) {
        // the largest logit that comes after (last, last_id) in the order (value descending, index ascending)
        float best = -INFINITY;
        int best_id = -1;
        for (int e = 0; e < E; ++e) {
            const float v = row[e];
            const bool after = v < last || (v == last && e > last_id);
            if (after && (best_id < 0 || v > best)) { best = v; best_id = e; }
        }
        if (best_id < 0) { best_id = 0; best = row[0]; }      // NaN logits: still a valid expert
        ids[(long long)t * top + s] = best_id;
        float w;
        if (weight_fn == 0) w = 1.0f / (1.0f + expf(-best));
        else { if (s == 0) zmax = best; w = expf(best - zmax); den += w; }
        wts[(long long)t * top + s] = w;
        last = best; last_id = best_id;
    }
    if (weight_fn == 1)
        for (int s = 0; s < top; ++s) wts[(long long)t * top + s] /= den;
}

// The limited choice of one token (see the head of the file).  row: its E logits; cs: E floats of scratch.
// Ties go to the lower index, among groups as among experts.  groups <= 64.
__device__ void choose_limited(const float* row, float* cs, int* ids, float* wts, long long t, int E, int top,
                               const float* corr, int groups, int keep, float scale) {
    for (int e = 0; e < E; ++e) cs[e] = 1.0f / (1.0f + expf(-row[e])) + (corr ? corr[e] : 0.f);
    const int per = E / groups;
    unsigned long long kept = ~0ull;
    if (keep < groups) {
        kept = 0ull;
        for (int r = 0; r < keep; ++r) {
            float best = -INFINITY;
            int best_g = -1;
            for (int g = 0; g < groups; ++g) {
                if ((kept >> g) & 1ull) continue;
                float m1 = -INFINITY, m2 = -INFINITY;             // the group's two largest
                for (int e = g * per; e < (g + 1) * per; ++e) {
                    const float v = cs[e];
                    if (v > m1) { m2 = m1; m1 = v; } else if (v > m2) m2 = v;
                }
                const float score = per > 1 ? m1 + m2 : m1;
                if (best_g < 0 || score > best) { best = score; best_g = g; }
            }
            kept |= 1ull << best_g;
        }
    }
    float last = INFINITY;
    int last_id = -1;
    for (int s = 0; s < top; ++s) {
        float best = -INFINITY;
        int best_id = -1;
        for (int e = 0; e < E; ++e) {
            if (!((kept >> (e / per)) & 1ull)) continue;
            const float v = cs[e];
            const bool after = v < last || (v == last && e > last_id);
            if (after && (best_id < 0 || v > best)) { best = v; best_id = e; }
        }
        if (best_id < 0) {                                       // NaN scores: still a valid expert, inside a kept group
            for (int e = 0; e < E && best_id < 0; ++e)
                if ((kept >> (e / per)) & 1ull) best_id = e;
            best = cs[best_id];
        }
        ids[(long long)t * top + s] = best_id;
        wts[(long long)t * top + s] = scale / (1.0f + expf(-row[best_id]));
        last = best; last_id = best_id;
    }
}

__global__ void route_kernel(const float* __restrict__ z, int stride, int* __restrict__ ids, float* __restrict__ wts,
                             int n_tokens, int E, int top, int weight_fn) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_tokens) return;
    choose(z + (long long)t * stride, ids, wts, t, E, top, weight_fn);
}

// Router logits and the choice in one kernel, a workgroup a token: z[t][n] = W[n] . h[t] in float32 (the
// lanes of a wave take every 64th term and add their sums in a fixed butterfly, so a token's logits do not
// depend on the step it is in), n < N rows of which the first E are experts (the rest: gates of other kinds
// that are wanted as float32 products of the same rows).
constexpr int ROUTER_WAVES = 16;

// TB tokens a workgroup: a wave keeps a piece of its row of W in registers for all of them, so the row is asked for
// once a workgroup.  A token's sums are the same chain whatever TB is.
template <typename T, int TB>
__global__ __launch_bounds__(ROUTER_WAVES * WAVE) void router_kernel(const T* __restrict__ h, const float* __restrict__ W,
                                                                      float* __restrict__ z, int* __restrict__ ids,
                                                                      float* __restrict__ wts, int n_tokens, int d, int N, int E, int top,
                                                                      int weight_fn, const float* __restrict__ bias,
                                                                      const float* __restrict__ corr, int groups, int keep, float scale) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    const int dp = (d + 3) & ~3;
    float* xs = sm;                                        // TB rows of d floats, each padded to a multiple of 4
    float* zs = sm + TB * dp;                              // TB rows of N logits
    float* cs = zs + TB * N;                               // a limited choice: TB rows of E choice scores
    const long long t0 = (long long)blockIdx.x * TB;
    const int nt = (int)min((long long)TB, n_tokens - t0);
    for (int b = 0; b < TB; ++b)
        for (int c = threadIdx.x; c < d; c += ROUTER_WAVES * WAVE) xs[b * dp + c] = b < nt ? to_f32(h[(t0 + b) * d + c]) : 0.f;
    __syncthreads();
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    for (int n = wave; n < N; n += ROUTER_WAVES) {
        const float* wr = W + (long long)n * d;
        float acc[TB];
#pragma unroll
        for (int b = 0; b < TB; ++b) acc[b] = 0.f;
        if (d % 4 == 0) {
            // four neighbouring terms a lane and step, several steps' loads under way at a time
#pragma unroll 8
            for (int c = lane * 4; c < d; c += 4 * WAVE) {
                const f32x4 w4 = *(const f32x4*)(wr + c);
#pragma unroll
                for (int b = 0; b < TB; ++b) {
                    const f32x4 x4 = *(const f32x4*)(xs + b * dp + c);
                    acc[b] = fmaf(w4[0], x4[0], acc[b]); acc[b] = fmaf(w4[1], x4[1], acc[b]);
                    acc[b] = fmaf(w4[2], x4[2], acc[b]); acc[b] = fmaf(w4[3], x4[3], acc[b]);
                }
            }
        } else {
#pragma unroll 8
            for (int c = lane; c < d; c += WAVE) {
                const float w = wr[c];
#pragma unroll
                for (int b = 0; b < TB; ++b) acc[b] = fmaf(w, xs[b * dp + c], acc[b]);
            }
        }
#pragma unroll
        for (int b = 0; b < TB; ++b) {
            float a = wave_sum(acc[b]);
            if (bias && n < E) a += bias[n];
            if (lane == 0 && b < nt) { zs[b * N + n] = a; z[(t0 + b) * N + n] = a; }
        }
    }
    __syncthreads();
    if (threadIdx.x < nt) {
        if (groups > 0) choose_limited(zs + threadIdx.x * N, cs + threadIdx.x * E, ids, wts, t0 + threadIdx.x, E, top, corr, groups, keep, scale);
        else choose(zs + threadIdx.x * N, ids, wts, t0 + threadIdx.x, E, top, weight_fn);
    }
}

constexpr int ROWS_WG = 16;          // output rows a workgroup of four waves computes

// a[row][f] = act(W_up[e][f] . x) (gated: glu(W_gate[e][f] . x, W_up[e][f] . x)), x = h[t] (times the choice's weight),
// rounded to T as the second product takes it
template <typename T>
__global__ __launch_bounds__(256) void expert_up_kernel(const T* __restrict__ h, const T* __restrict__ w_up, const int* __restrict__ ids,
                                                        const float* __restrict__ wts, T* __restrict__ a, int d, int F, int top,
                                                        int act, int scale_input, int gated, float limit, float alpha) {
    extern __shared__ float xs[];
    const long long row = blockIdx.x;
    const long long t = row / top;
    const int e = ids[row];
    const float w = scale_input ? wts[row] : 1.f;
    for (int c = threadIdx.x; c < d; c += 256) xs[c] = to_f32(from_f32<T>(to_f32(h[t * d + c]) * w));
    __syncthreads();
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    for (int f = blockIdx.y * ROWS_WG + wave; f < min(F, (int)(blockIdx.y + 1) * ROWS_WG); f += 4) {
        // gated: the expert's first matrices lie one after the other, gate [F][d] then up [F][d]
        const T* wr = w_up + ((long long)e * (gated ? 2 * F : F) + f) * d;
        float acc = 0.f;
        for (int c = lane; c < d; c += WAVE) acc = fmaf(to_f32(wr[c]), xs[c], acc);
        acc = wave_sum(acc);
        float res;
        if (gated) {
            const T* wu = wr + (long long)F * d;
            float up = 0.f;
            for (int c = lane; c < d; c += WAVE) up = fmaf(to_f32(wu[c]), xs[c], up);
            res = glu_fn(acc, wave_sum(up), act, limit, alpha);
        } else res = act_fn(acc, act);
        if (lane == 0) a[row * F + f] = from_f32<T>(res);
    }
}

// y[row][c] = W_down[e][c] . a[row]  (float32)
template <typename T>
__global__ __launch_bounds__(256) void expert_down_kernel(const T* __restrict__ a, const T* __restrict__ w_down, const int* __restrict__ ids,
                                                          float* __restrict__ y, int d, int F) {
    extern __shared__ float as[];
    const long long row = blockIdx.x;
    const int e = ids[row];
    for (int f = threadIdx.x; f < F; f += 256) as[f] = to_f32(a[row * F + f]);
    __syncthreads();
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    for (int c = blockIdx.y * ROWS_WG + wave; c < min(d, (int)(blockIdx.y + 1) * ROWS_WG); c += 4) {
        const T* wr = w_down + ((long long)e * d + c) * F;
        float acc = 0.f;
        for (int f = lane; f < F; f += WAVE) acc = fmaf(to_f32(wr[f]), as[f], acc);
        acc = wave_sum(acc);
        if (lane == 0) y[row * d + c] = acc;
    }
}

// residual[t][c] += sum over the token's choices, in their order, of y[t * top + s][c] (times the weight)
__global__ void combine_kernel(const float* __restrict__ y, const float* __restrict__ wts, float* __restrict__ residual,
                               long long n, int d, int top, int scale_output) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const long long t = i / d;
    const int c = (int)(i - t * d);
    float acc = 0.f;
    for (int s = 0; s < top; ++s) {
        const float v = y[(t * top + s) * d + c];
        acc += scale_output ? v * wts[t * top + s] : v;
    }
    residual[i] += acc;
}

// ------------------------------------------------------------ many rows: grouped by expert, matrix cores
typedef __bf16 bf16x8_ __attribute__((ext_vector_type(8)));
constexpr int GROUP_MAX_E = 1024;

// One workgroup sorts the rows (token, choice) by expert and cuts each expert's rows into tiles of TM:
// sorted[pos] = row; tiles[i] = (expert, first pos, rows), expert -1 for tiles beyond the last.  The order of an
// expert's rows among themselves is whatever the atomics give: no row's result depends on its place in a tile.
__global__ __launch_bounds__(1024) void group_rows_kernel(const int* __restrict__ ids, int R, int E, int TM, int* __restrict__ sorted,
                                                          int* __restrict__ tiles, int max_tiles) {
    __shared__ int cnt[GROUP_MAX_E], off[GROUP_MAX_E], cur[GROUP_MAX_E];
    for (int e = threadIdx.x; e < E; e += 1024) { cnt[e] = 0; cur[e] = 0; }
    __syncthreads();
    for (int r = threadIdx.x; r < R; r += 1024) atomicAdd(&cnt[ids[r]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int o = 0, nt = 0;
        for (int e = 0; e < E; ++e) {
            off[e] = o;
            for (int p = 0; p < cnt[e] && nt < max_tiles; p += TM, ++nt) {
                tiles[3 * nt] = e; tiles[3 * nt + 1] = o + p; tiles[3 * nt + 2] = min(TM, cnt[e] - p);
            }
            o += cnt[e];
        }
        for (; nt < max_tiles; ++nt) { tiles[3 * nt] = -1; tiles[3 * nt + 1] = 0; tiles[3 * nt + 2] = 0; }
    }
    __syncthreads();
    for (int r = threadIdx.x; r < R; r += 1024) {
        const int e = ids[r];
        sorted[off[e] + atomicAdd(&cur[e], 1)] = r;
    }
}

__device__ __forceinline__ f32x4 mfma16(bf16x8_ a, bf16x8_ b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// A tile of up to 16 TMT rows of one expert times a slice of that expert's matrix.  W: every expert's matrix
// [N][K] in blocks of 16 rows x 32 k in the order of the matrix cores' first operand ([E][ceil(N/16)][ceil(K/32)]
// blocks of 1 KB: piece l = row l % 16, k 8 (l / 16) .. + 7); a wave takes NF blocks of rows, the four waves of a
// workgroup neighbouring ones.  UP: the rows are tokens of h gathered through `sorted` (row / top), times the
// choice's weight and rounded where scale_input; the result act(.) goes to A [R][N] in sorted order.  Else: the
// rows are A's, in place, and the float32 result goes to Y [R][N] at the row's own number.
template <int NF, int TMT, bool UP>
__global__ __launch_bounds__(256) void grouped_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                      const int* __restrict__ tiles, const int* __restrict__ sorted,
                                                      const float* __restrict__ wts, bf16_t* __restrict__ A, float* __restrict__ Y,
                                                      int K, int N, int top, int act, int scale_input, int gated, float limit,
                                                      float alpha) {
    const int tile = blockIdx.x;
    const int e = tiles[3 * tile];
    if (e < 0) return;
    const int pos0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, n16 = lane % 16, g = lane / 16;
    const int NT16 = (N + 15) / 16, KB = (K + 31) / 32;
    const int ft0 = (blockIdx.y * 4 + wave) * NF;
    if (ft0 >= NT16) return;
    long long src[TMT];
    int own[TMT];
    float scale[TMT];
    bool valid[TMT];
#pragma unroll
    for (int tt = 0; tt < TMT; ++tt) {
        const int idx = tt * 16 + n16;
        valid[tt] = idx < rows;
        own[tt] = valid[tt] ? sorted[pos0 + idx] : 0;
        src[tt] = UP ? own[tt] / top : pos0 + idx;
        scale[tt] = (UP && scale_input && valid[tt]) ? wts[own[tt]] : 1.f;
    }
    f32x4 acc[NF][TMT];
#pragma unroll
    for (int nf = 0; nf < NF; ++nf)
#pragma unroll
        for (int tt = 0; tt < TMT; ++tt) acc[nf][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
    const bf16x8_ zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const bf16_t* We = W + (long long)e * NT16 * KB * 512;
    constexpr int UN = NF == 1 ? 8 : 4;        // few registers a step: more loads under way (narrow tiles stream the weights)
#pragma unroll UN
    for (int kb = 0; kb < KB; ++kb) {
        const int k = kb * 32 + 8 * g;
        bf16x8_ xb[TMT];
#pragma unroll
        for (int tt = 0; tt < TMT; ++tt) {
            xb[tt] = (valid[tt] && k < K) ? *(const bf16x8_*)(X + src[tt] * K + k) : zero;
            if (UP && scale_input) {
#pragma unroll
                for (int i = 0; i < 8; ++i) xb[tt][i] = (bf16_t)((float)xb[tt][i] * scale[tt]);
            }
        }
#pragma unroll
        for (int nf = 0; nf < NF; ++nf) {
            if (ft0 + nf < NT16) {
                const bf16x8_ wa = *(const bf16x8_*)(We + (((long long)(ft0 + nf) * KB + kb) * 64 + lane) * 8);
#pragma unroll
                for (int tt = 0; tt < TMT; ++tt) acc[nf][tt] = mfma16(wa, xb[tt], acc[nf][tt]);
            }
        }
    }
#pragma unroll
    for (int nf = 0; nf < NF; ++nf)
#pragma unroll
        for (int tt = 0; tt < TMT; ++tt) {
            if (!valid[tt] || ft0 + nf >= NT16) continue;
            const int col = (ft0 + nf) * 16 + 4 * g;
            if (UP && gated) {
                // rows 2f and 2f + 1 of the first matrix are feature f's gate and up: a lane holds two features
#pragma unroll
                for (int i = 0; i < 4; i += 2)
                    if (col + i + 1 < N)
                        A[(long long)(pos0 + tt * 16 + n16) * (N / 2) + (col + i) / 2] =
                            (bf16_t)glu_fn(acc[nf][tt][i], acc[nf][tt][i + 1], act, limit, alpha);
                continue;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (col + i >= N) continue;
                if (UP) A[(long long)(pos0 + tt * 16 + n16) * N + col + i] = (bf16_t)act_fn(acc[nf][tt][i], act);
                else Y[(long long)own[tt] * N + col + i] = acc[nf][tt][i];
            }
        }
}
}  // namespace

TUFF_EXPORT int tuff_moe_route(const float* z, int stride, int* ids, float* wts, int n_tokens, int E, int top, int weight_fn,
                               hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (top < 1 || top > E || stride < E) return -2;
    hipLaunchKernelGGL(route_kernel, dim3(ceil_div(n_tokens, 64)), dim3(64), 0, stream, z, stride, ids, wts, n_tokens, E, top, weight_fn);
    return launch_status();
}

// h [T][d], w_up [E][F][d] (gated: [E][2 F][d], an expert's gate rows then its up rows), w_down [E][d][F] of type dt; ids, wts [T][top]; a [T*top][F] (type dt) and
// y [T*top][d] (float32) are work arrays; residual float32 [T][d].
TUFF_EXPORT int tuff_moe_experts(const void* h, const void* w_up, const void* w_down, int dt, const int* ids, const float* wts,
                                 void* a, float* y, float* residual, int n_tokens, int d, int F, int top, int act,
                                 int scale_input, int gated, float limit, float alpha, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (d > 16384 || F > 16384) return -2;
    const long long rows = (long long)n_tokens * top;
    dim3 block(256);
    if (dt == DT_F32) {
        hipLaunchKernelGGL(expert_up_kernel<float>, dim3((unsigned)rows, ceil_div(F, ROWS_WG)), block, d * sizeof(float), stream,
                           (const float*)h, (const float*)w_up, ids, wts, (float*)a, d, F, top, act, scale_input, gated, limit, alpha);
        hipLaunchKernelGGL(expert_down_kernel<float>, dim3((unsigned)rows, ceil_div(d, ROWS_WG)), block, F * sizeof(float), stream,
                           (const float*)a, (const float*)w_down, ids, y, d, F);
    } else {
        hipLaunchKernelGGL(expert_up_kernel<bf16_t>, dim3((unsigned)rows, ceil_div(F, ROWS_WG)), block, d * sizeof(float), stream,
                           (const bf16_t*)h, (const bf16_t*)w_up, ids, wts, (bf16_t*)a, d, F, top, act, scale_input, gated, limit, alpha);
        hipLaunchKernelGGL(expert_down_kernel<bf16_t>, dim3((unsigned)rows, ceil_div(d, ROWS_WG)), block, F * sizeof(float), stream,
                           (const bf16_t*)a, (const bf16_t*)w_down, ids, y, d, F);
    }
    const long long n = (long long)n_tokens * d;
    hipLaunchKernelGGL(combine_kernel, dim3((unsigned)ceil_div_ll(n, 256)), block, 0, stream, y, wts, residual, n, d, top, !scale_input);
    return launch_status();
}

// z float32 [T][N], the first E columns the experts' logits; ids, wts [T][top].  W float32 [N][d]; h [T][d] of type dt.
// bias float32 [E] or null: added to the experts' logits before the choice.  groups > 0: the limited choice (weight_fn 0),
// with corr float32 [E] or null, `keep` of `groups` groups and the weights times `scale`; groups 0: the plain choice.
TUFF_EXPORT int tuff_moe_router(const void* h, int dt, const float* W, float* z, int* ids, float* wts, int n_tokens, int d,
                                int N, int E, int top, int weight_fn, const float* bias, const float* corr, int groups, int keep,
                                float scale, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    const int extra = groups > 0 ? E : 0;
    if (top < 1 || top > E || N < E || (long long)(d + 4 + N + extra) * 4 > 65536) return -2;
    if (groups > 0 && (weight_fn != 0 || groups > 64 || E % groups || keep < 1 || keep > groups || top > keep * (E / groups))) return -2;
    // long steps: four tokens a workgroup where that fits the LDS (the rows of W are then read a quarter as often)
    const bool four = n_tokens >= 1024 && (long long)(d + 4 + N + extra) * 16 <= 65536;
    const int TB = four ? 4 : 1;
    const size_t lds = (size_t)TB * (((d + 3) & ~3) + N + extra) * sizeof(float);
    const dim3 grid((unsigned)ceil_div(n_tokens, TB)), block(ROUTER_WAVES * WAVE);
#define LAUNCH(T, B) hipLaunchKernelGGL((router_kernel<T, B>), grid, block, lds, stream, (const T*)h, W, z, ids, wts, n_tokens, d, N, E, top, weight_fn, bias, corr, groups, keep, scale)
    if (dt == DT_F32) { if (four) LAUNCH(float, 4); else LAUNCH(float, 1); }
    else { if (four) LAUNCH(bf16_t, 4); else LAUNCH(bf16_t, 1); }
#undef LAUNCH
    return launch_status();
}

// The experts of steps with many rows an expert: block tiles of 128 rows of one expert x 128 rows of its matrix, the
// operands of a step of 64 k staged through LDS and shared by the workgroup's eight waves (2 x 4, each 64 rows x 32
// features as 4 x 2 products), so an expert's matrix is read once for 128 rows where grouped_kernel reads it once for
// 32.  Two LDS buffers: while a step is multiplied out of one, the next step's operands travel from memory into
// registers and then into the other; one barrier a step.  X rows lie in LDS row-major with their 16-byte chunks
// exchanged (chunk c of row r at position c ^ (r % 8)), W as in memory (1 KB blocks, lane l's operand at 16 l).
// The products of a row run over k in ascending steps of 32 with one accumulator, as in grouped_kernel: the two
// kernels give the same bits, and a row's result does not depend on its tile.
constexpr int GT_BM = 128, GT_BN = 128, GT_BK = 64, GT_NT = 512;

__device__ __forceinline__ int gt_swz(int r, int c) { return r * GT_BK + ((c ^ (r % 8)) * 8); }

template <bool UP>
__global__ __launch_bounds__(GT_NT) void grouped_tiled_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                              const int* __restrict__ tiles, const int* __restrict__ sorted,
                                                              const float* __restrict__ wts, bf16_t* __restrict__ A,
                                                              float* __restrict__ Y, int K, int N, int top, int act, int scale_input,
                                                              int gated, float limit, float alpha) {
    extern __shared__ __attribute__((aligned(16))) bf16_t gt_lds[];     // [2][BM * BK] of X, then [2][BN * BK] of W
    const int tile = blockIdx.x;
    const int e = tiles[3 * tile];
    if (e < 0) return;
    const int pos0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
    const int n0 = blockIdx.y * GT_BN;
    const int NT16 = (N + 15) / 16, KB = (K + 31) / 32;
    bf16_t* As = gt_lds;
    bf16_t* Bs = gt_lds + 2 * GT_BM * GT_BK;
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE, r16 = lane % 16, g = lane / 16;
    const int wm = (wave / 4) * 64, wn = (wave % 4) * 32;

    // what this thread moves a step: two 16-byte pieces of X (rows tid / 8 and 64 further, chunk tid % 8) and two of
    // W (piece tid % 64 of block (tid / 64) % 2 ... of row tiles tid / 128 and 4 further).  Rows beyond the tile's
    // read its first row, row tiles beyond the matrix its last: their results are never stored.
    const int c0 = tid % 8;
    const bf16_t* xsrc[2];
    int xdst[2];
    float xscale[2];                                           // UP with scale_input: the choice's weight on the row's input
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int r = tid / 8 + p * 64;
        const int rr = r < rows ? r : 0;
        const long long row = UP ? sorted[pos0 + rr] / top : pos0 + rr;
        xscale[p] = (UP && scale_input) ? wts[sorted[pos0 + rr]] : 1.f;
        xsrc[p] = X + row * K + c0 * 8;
        xdst[p] = gt_swz(r, c0);
    }
    const int wpiece = tid % 64, wh = (tid / 64) % 2;
    const bf16_t* We = W + (long long)e * NT16 * KB * 512;
    const bf16_t* wsrc[2];
    int wdst[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int t = tid / 128 + p * 4;                       // row tile of the block, 0 .. 7
        const int tt = min(n0 / 16 + t, NT16 - 1);
        wsrc[p] = We + ((long long)tt * KB + wh) * 512 + wpiece * 8;
        wdst[p] = (t * 2 + wh) * 512 + wpiece * 8;
    }
    const bf16x8_ zero = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8_ rx[2], rw[2];
    auto load = [&](int kt) {
        const int k0 = kt * GT_BK;
        const bool in_x = k0 + c0 * 8 < K, in_w = k0 / 32 + wh < KB;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            rx[p] = in_x ? *(const bf16x8_*)(xsrc[p] + k0) : zero;
            if (UP && scale_input) {
#pragma unroll
                for (int i = 0; i < 8; ++i) rx[p][i] = (bf16_t)((float)rx[p][i] * xscale[p]);
            }
            rw[p] = in_w ? *(const bf16x8_*)(wsrc[p] + (long long)(k0 / 32) * 512) : zero;
        }
    };
    auto store = [&](int buf) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            *(bf16x8_*)(As + buf * GT_BM * GT_BK + xdst[p]) = rx[p];
            *(bf16x8_*)(Bs + buf * GT_BN * GT_BK + wdst[p]) = rw[p];
        }
    };
    f32x4 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int nk = (K + GT_BK - 1) / GT_BK;
    load(0);
    store(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) load(kt + 1);
        const bf16_t* Ab = As + buf * GT_BM * GT_BK;
        const bf16_t* Bb = Bs + buf * GT_BN * GT_BK;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            bf16x8_ b[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) b[j] = *(const bf16x8_*)(Bb + ((wn / 16 + j) * 2 + half) * 512 + lane * 8);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bf16x8_ a = *(const bf16x8_*)(Ab + gt_swz(wm + i * 16 + r16, half * 4 + g));
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = mfma16(b[j], a, acc[i][j]);
            }
        }
        if (kt + 1 < nk) store(buf ^ 1);
        __syncthreads();
    }

    // acc[i][j][q]: row wm + 16 i + r16 of the tile, column n0 + wn + 16 j + 4 g + q
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = wm + i * 16 + r16;
        if (r >= rows) continue;
        const long long own = UP ? 0 : sorted[pos0 + r];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = n0 + wn + j * 16 + 4 * g;
            if (col >= N) continue;
            const f32x4 v = acc[i][j];
            if (UP && gated) {
                // rows 2f and 2f + 1 of the first matrix are feature f's gate and up
#pragma unroll
                for (int q = 0; q < 4; q += 2)
                    if (col + q + 1 < N)
                        A[(long long)(pos0 + r) * (N / 2) + (col + q) / 2] = (bf16_t)glu_fn(v[q], v[q + 1], act, limit, alpha);
            } else if (UP) {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (col + q < N) A[(long long)(pos0 + r) * N + col + q] = (bf16_t)act_fn(v[q], act);
            } else if (col + 3 < N && N % 4 == 0) {
                *(f32x4*)(Y + own * N + col) = v;
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (col + q < N) Y[own * N + col + q] = v[q];
            }
        }
    }
}

// From which width of both matrices on (rows of the first, rows of the second) steps with many rows an expert take
// tiles of 64 rows.  Measured, 2,048 tokens with gated experts: hidden size 4,096, 32 experts of 1,536, four chosen:
// 1.25 ms against 1.62 ms with tiles of 32; hidden size 2,048, 16 experts of 1,024, two chosen: 0.33 against 0.31.
// For measurements and tests; the result does not depend on it.  Returns the value before.
static int wide_from = 4096;
// From how many rows an expert (on average over the step) on the experts run in block tiles of 128 rows through LDS.
// For measurements and tests; the result does not depend on it.  Returns the value before.
static int tiled_from = 96;
TUFF_EXPORT int tuff_moe_grouped_tiled_from(int n) {
    const int old = tiled_from;
    if (n >= 0) tiled_from = n;
    return old;
}

TUFF_EXPORT int tuff_moe_grouped_wide_from(int n) {
    const int old = wide_from;
    if (n >= 0) wide_from = n;
    return old;
}

// Rows a tile of tuff_moe_experts_grouped holds for R rows over E experts, and the tiles it may need.
TUFF_EXPORT int tuff_moe_grouped_tile_rows(long long R, int E) { return R >= 24ll * E ? 32 : 16; }

// The experts of many rows on the matrix cores (bfloat16): h [T][d]; w_up, w_down every expert's matrix in blocks
// (see grouped_kernel), [E][F x d] and [E][d x F]; ids, wts [T][top]; work arrays sorted int32 [T*top], tiles int32
// [3 * max_tiles] with max_tiles >= ceil(T*top / tile rows) + E, a bfloat16 [T*top][F], y float32 [T*top][d];
// residual float32 [T][d].  d and F multiples of 8, E at most 1024.  gated: w_up is [E][2 F x d] with row 2 f feature
// f's gate row and row 2 f + 1 its up row.
TUFF_EXPORT int tuff_moe_experts_grouped(const void* h, const void* w_up, const void* w_down, const int* ids, const float* wts,
                                         int* sorted, int* tiles, int max_tiles, void* a, float* y, float* residual,
                                         int n_tokens, int d, int F, int E, int top, int act, int scale_input, int gated,
                                         float limit, float alpha, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    const long long R = (long long)n_tokens * top;
    if (d % 8 || F % 8 || E > GROUP_MAX_E || E < 1 || R > 0x7fffffffll) return -2;
    int TM = tuff_moe_grouped_tile_rows(R, E);
    if (max_tiles < (int)((R + TM - 1) / TM) + E) return -2;
    const int F1 = gated ? 2 * F : F;        // rows of the first matrix (gated: gate and up rows take turns)
    // Many rows an expert and matrices wide enough to fill the chip with fewer, taller tiles: 64 rows a tile, so an
    // expert's matrix is read half as often (the caller's tile array, sized for 32 rows, is more than enough).
    if (TM == 32 && R >= 128ll * E && F1 >= wide_from && d >= wide_from) TM = 64;
    const bf16_t* H_ = (const bf16_t*)h;
    bf16_t* A_ = (bf16_t*)a;
    // Many rows an expert: block tiles of 128 rows through LDS (the caller's tile array is sized for smaller tiles and
    // holds these).
    if (R >= (long long)tiled_from * E) {
        constexpr int lds = 2 * (GT_BM + GT_BN) * GT_BK * 2;
        static bool set = false;
        if (!set) {
            if (hipFuncSetAttribute((const void*)grouped_tiled_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess ||
                hipFuncSetAttribute((const void*)grouped_tiled_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
                return -1;
            set = true;
        }
        hipLaunchKernelGGL(group_rows_kernel, dim3(1), dim3(1024), 0, stream, ids, (int)R, E, GT_BM, sorted, tiles, max_tiles);
        hipLaunchKernelGGL(grouped_tiled_kernel<true>, dim3(max_tiles, ceil_div(F1, GT_BN)), dim3(GT_NT), lds, stream,
                           H_, (const bf16_t*)w_up, tiles, sorted, wts, A_, nullptr, d, F1, top, act, scale_input, gated, limit, alpha);
        hipLaunchKernelGGL(grouped_tiled_kernel<false>, dim3(max_tiles, ceil_div(d, GT_BN)), dim3(GT_NT), lds, stream,
                           A_, (const bf16_t*)w_down, tiles, sorted, wts, nullptr, y, F, d, top, act, 0, 0, 0.f, 0.f);
        const long long n = (long long)n_tokens * d;
        hipLaunchKernelGGL(combine_kernel, dim3((unsigned)ceil_div_ll(n, 256)), dim3(256), 0, stream, y, wts, residual, n, d, top, !scale_input);
        return launch_status();
    }
    hipLaunchKernelGGL(group_rows_kernel, dim3(1), dim3(1024), 0, stream, ids, (int)R, E, TM, sorted, tiles, max_tiles);
    // few rows an expert: many narrow workgroups stream the weights; many: wide ones reuse them
    if (TM == 64) {
        hipLaunchKernelGGL((grouped_kernel<4, 4, true>), dim3(max_tiles, ceil_div(ceil_div(F1, 16), 16)), dim3(256), 0, stream,
                           H_, (const bf16_t*)w_up, tiles, sorted, wts, A_, nullptr, d, F1, top, act, scale_input, gated, limit, alpha);
        hipLaunchKernelGGL((grouped_kernel<4, 4, false>), dim3(max_tiles, ceil_div(ceil_div(d, 16), 16)), dim3(256), 0, stream,
                           A_, (const bf16_t*)w_down, tiles, sorted, wts, nullptr, y, F, d, top, act, scale_input, 0, 0.f, 0.f);
    } else if (TM == 32) {
        hipLaunchKernelGGL((grouped_kernel<4, 2, true>), dim3(max_tiles, ceil_div(ceil_div(F1, 16), 16)), dim3(256), 0, stream,
                           H_, (const bf16_t*)w_up, tiles, sorted, wts, A_, nullptr, d, F1, top, act, scale_input, gated, limit, alpha);
        hipLaunchKernelGGL((grouped_kernel<4, 2, false>), dim3(max_tiles, ceil_div(ceil_div(d, 16), 16)), dim3(256), 0, stream,
                           A_, (const bf16_t*)w_down, tiles, sorted, wts, nullptr, y, F, d, top, act, scale_input, 0, 0.f, 0.f);
    } else {
        hipLaunchKernelGGL((grouped_kernel<1, 1, true>), dim3(max_tiles, ceil_div(ceil_div(F1, 16), 4)), dim3(256), 0, stream,
                           H_, (const bf16_t*)w_up, tiles, sorted, wts, A_, nullptr, d, F1, top, act, scale_input, gated, limit, alpha);
        hipLaunchKernelGGL((grouped_kernel<1, 1, false>), dim3(max_tiles, ceil_div(ceil_div(d, 16), 4)), dim3(256), 0, stream,
                           A_, (const bf16_t*)w_down, tiles, sorted, wts, nullptr, y, F, d, top, act, scale_input, 0, 0.f, 0.f);
    }
    const long long n = (long long)n_tokens * d;
    hipLaunchKernelGGL(combine_kernel, dim3((unsigned)ceil_div_ll(n, 256)), dim3(256), 0, stream, y, wts, residual, n, d, top, !scale_input);
    return launch_status();
}
