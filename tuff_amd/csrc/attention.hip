// Attention of a mixed batch over the paged cache: every token of the step, prompt
// portion or decoded token alike, attends to the keys of its own request at positions
// lo..pos, lo = 0 or pos - window + 1, read from the pages its block table names.  The
// step's own keys were written to the cache before this runs, so nothing but the cache
// is read (cf. src/lfm25_engine.c:552-568: all K/V of a batch are written before any
// attention, and token j is bounded by its own position).
//
// Scores are scaled by 1/sqrt(hd); softmax is the running-max form of
// src/lfm25_gpu.cu:531-555 over key tiles of 64; query head h reads kv head
// h / (H / Hkv).  Scores, softmax and the weighted sum are float32.  The key tiles are
// aligned to absolute positions (0, 64, 128, ...), so the order of every sum depends
// only on the token's position, not on how the sequence was cut into steps.
//
// Cache layout: K [page][kv_head][offset][hd], V [page][kv_head][hd][offset].
//
// Values may be of another width than keys (vd; V [page][kv_head][vd][offset]), and a head may
// have a sink: a learned logit whose exponential counts once in the softmax's denominator and
// that has neither key nor value (it is not scaled).
//
// A head may also have a distance slope: slope_h * (pos - key) is taken off the scaled score (from
// the integer distance, so that far positions lose no bits).  And the values may be the leading vd
// channels of the key rows themselves (v_in_k: a cache of one latent row a position that serves as key
// and value; v_cache is then not read).
//
// Or a logarithmic distance penalty: r1_h * ln(1 + r2_h * (pos - key)) is taken off the scaled score.
// And a query head's weights may be applied to the values of every kv head (all_v: the third grid axis
// is the kv head whose values are read, out is [token][head][kv head][vd]); mixing the heads' softmax
// weights is linear in them, so a kernel that follows forms the mixed heads from these sums.
//
// This is the general kernel: any head size up to 640, any page size, float32 or
// bfloat16 cache.  One wave per (token, head): lanes are keys for q.k, lanes are
// channels for p.v.
#include "common.h"
#include <math.h>

namespace {
constexpr int MAX_PER_LANE_WIDE = 10;

template <typename T, int MAX_PER_LANE>
__global__ __launch_bounds__(WAVE) void attention_general_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache, T* __restrict__ out,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ req_of_token,
    const int* __restrict__ positions, int H, int Hkv, int hd, int vd, int page_size, int window, float scale, const float* __restrict__ sinks,
    const float* __restrict__ slopes, int v_in_k, const float* __restrict__ log_r1, const float* __restrict__ log_r2,
    int all_v) {
    __shared__ float qs[MAX_PER_LANE * WAVE];
    __shared__ float ps[WAVE];
    __shared__ long long voff[WAVE];
    const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int kvh = head / (H / Hkv);
    const int pos = positions[t];
    const int lo = (window > 0) ? max(0, pos - window + 1) : 0;
    const int* table = block_table + (long long)req_of_token[t] * max_blocks;
    const T* qrow = q + ((long long)t * H + head) * hd;
    const float slope = slopes ? slopes[head] : 0.f;
    const float r1 = log_r1 ? log_r1[head] : 0.f, r2 = log_r1 ? log_r2[head] : 0.f;
    const int vh = all_v ? blockIdx.z : kvh;                  // the kv head whose values are read
    const T* v_base = v_in_k ? k_cache : v_cache;
    const long long v_step = v_in_k ? 1 : page_size;          // from a value's channel to the next
    for (int j = lane; j < hd; j += WAVE) qs[j] = to_f32(qrow[j]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[MAX_PER_LANE];
#pragma unroll
    for (int i = 0; i < MAX_PER_LANE; ++i) acc[i] = 0.f;

    for (int t0 = (lo / WAVE) * WAVE; t0 <= pos; t0 += WAVE) {
        const int kt = t0 + lane;
        const bool valid = kt >= lo && kt <= pos;
        float s = -INFINITY;
        long long base = 0;
        if (valid) {
            const long long page = table[kt / page_size];
            const long long head_base = (page * Hkv + kvh) * page_size;
            base = v_in_k ? head_base * hd + (long long)(kt % page_size) * hd      // the key's own row
                          : (page * Hkv + vh) * page_size * vd + (kt % page_size); // V: [vd][page_size], this key's column
            const T* krow = k_cache + head_base * hd + (long long)(kt % page_size) * hd;
            float d = 0.f;
            for (int j = 0; j < hd; ++j) d = fmaf(qs[j], to_f32(krow[j]), d);
            s = d * scale - slope * (float)(pos - kt);
            if (log_r1) s -= r1 * log1pf(r2 * (float)(pos - kt));
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);          // 0 on the first tile (m = -inf)
        l = l * corr + wave_sum(p);
        m = m_new;
        __syncthreads();                             // previous tile's ps/voff fully consumed
        ps[lane] = p;
        voff[lane] = base;
        __syncthreads();
        const int n_keys = min(WAVE, pos - t0 + 1);
#pragma unroll
        for (int i = 0; i < MAX_PER_LANE; ++i) acc[i] *= corr;
        for (int jj = 0; jj < n_keys; ++jj) {
            const float pj = ps[jj];
            if (pj == 0.f) continue;                 // masked (below the window) or underflowed
            const T* vcol = v_base + voff[jj];
#pragma unroll
            for (int i = 0; i < MAX_PER_LANE; ++i) {
                const int j = lane + i * WAVE;
                if (j < vd) acc[i] = fmaf(pj, to_f32(vcol[(long long)j * v_step]), acc[i]);
            }
        }
    }
    T* o = out + ((long long)t * H + head) * vd;
    // (all_v: float32 sums whatever the compute type, for the kernel that mixes the heads)
    float* o_wide = (float*)out + (((long long)t * H + head) * Hkv + vh) * vd;
    float keep = 1.f;
    if (sinks) {
        // the sink joins the denominator under the common maximum
        const float sk = sinks[head];
        const float m_new = fmaxf(m, sk);
        keep = expf(m - m_new);
        l = l * keep + expf(sk - m_new);
    }
    const float inv = keep / l;
#pragma unroll
    for (int i = 0; i < MAX_PER_LANE; ++i) {
        const int j = lane + i * WAVE;
        if (j < vd) {
            if (all_v) o_wide[j] = acc[i] * inv;
            else o[j] = from_f32<T>(acc[i] * inv);
        }
    }
}
}  // namespace

TUFF_EXPORT int tuff_attention_general(const void* q, const void* k_cache, const void* v_cache, void* out, int dt,
                                       const int* block_table, int max_blocks, const int* req_of_token,
                                       const int* positions, int n_tokens, int H, int Hkv, int hd, int vd, int page_size,
                                       int window, float scale, const float* sinks, const float* slopes, int v_in_k,
                                       const float* log_r1, const float* log_r2, int all_v, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    const int widest = max(hd, vd);
    if (widest > MAX_PER_LANE_WIDE * WAVE || vd <= 0 || Hkv <= 0 || H % Hkv != 0 || (v_in_k && vd > hd)) return -2;
    if ((log_r1 == nullptr) != (log_r2 == nullptr) || (all_v && v_in_k) || H > 65535 || Hkv > 65535) return -2;
    dim3 grid(n_tokens, H, all_v ? Hkv : 1), block(WAVE);
#define LAUNCH(T, PL) hipLaunchKernelGGL((attention_general_kernel<T, PL>), grid, block, 0, stream, (const T*)q, (const T*)k_cache, \
        (const T*)v_cache, (T*)out, block_table, max_blocks, req_of_token, positions, H, Hkv, hd, vd, page_size, window, scale, \
        sinks, slopes, v_in_k, log_r1, log_r2, all_v)
    if (widest <= 4 * WAVE) { if (dt == DT_F32) LAUNCH(float, 4); else LAUNCH(bf16_t, 4); }
    else { if (dt == DT_F32) LAUNCH(float, MAX_PER_LANE_WIDE); else LAUNCH(bf16_t, MAX_PER_LANE_WIDE); }
#undef LAUNCH
    return launch_status();
}

// After attention: the heads' softmax weights mixed and a gate per head, on the weighted sums.
//   all_v:  out[t][h][j] = gate(t, h) * sum_g talk[h][g] * o[t][g][kv(h)][j]     (o [T][H][Hkv][vd] float32)
//   else:   out[t][h][j] = gate(t, h) * o[t][h][j]                                (o [T][H][vd] of the compute type)
// gate(t, h) = sigmoid(gates[t * gate_stride + h]) (float32), or 1 without gates.  A wave a (token, head); the sum
// over g runs in ascending order.
namespace {
template <typename TI, typename T>
__global__ __launch_bounds__(WAVE) void head_mix_gate_kernel(const TI* __restrict__ o, const float* __restrict__ talk,
                                                             const float* __restrict__ gates, int gate_stride,
                                                             T* __restrict__ out, int H, int Hkv, int vd) {
    const long long t = blockIdx.x;
    const int h = blockIdx.y;
    const float g = gates ? 1.0f / (1.0f + expf(-gates[t * gate_stride + h])) : 1.f;
    T* dst = out + (t * H + h) * vd;
    if (talk) {
        const int kvh = h / (H / Hkv);
        for (int j = threadIdx.x; j < vd; j += WAVE) {
            float acc = 0.f;
            for (int q = 0; q < H; ++q) acc = fmaf(talk[h * H + q], to_f32(o[((t * H + q) * Hkv + kvh) * vd + j]), acc);
            dst[j] = from_f32<T>(acc * g);
        }
    } else {
        const TI* src = o + (t * H + h) * vd;
        for (int j = threadIdx.x; j < vd; j += WAVE) dst[j] = from_f32<T>(to_f32(src[j]) * g);
    }
}
}  // namespace

// in_dt: type of o; dt: type of out.  talk float32 [H][H] or null; gates float32 or null.
TUFF_EXPORT int tuff_head_mix_gate(const void* o, int in_dt, const float* talk, const float* gates, int gate_stride, void* out,
                                   int dt, int n_tokens, int H, int Hkv, int vd, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (H <= 0 || Hkv <= 0 || H % Hkv || H > 65535 || vd <= 0) return -2;
    dim3 grid(n_tokens, H), block(WAVE);
#define LAUNCH(TI, T) hipLaunchKernelGGL((head_mix_gate_kernel<TI, T>), grid, block, 0, stream, (const TI*)o, talk, gates, gate_stride, (T*)out, H, Hkv, vd)
    if (in_dt == DT_F32 && dt == DT_F32) LAUNCH(float, float);
    else if (in_dt == DT_F32) LAUNCH(float, bf16_t);
    else if (dt == DT_BF16) LAUNCH(bf16_t, bf16_t);
    else return -2;
#undef LAUNCH
    return launch_status();
}
