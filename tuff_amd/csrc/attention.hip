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

// ---------------------------------------------------------------------------------------------------------------
// Single tokens over a bfloat16 cache with float32 weights, in three kernels, so that the keys and the values of a
// request are read once whatever the number of query heads:
//   scores   a workgroup a (token, kv head, part of 256 keys), a thread a key: the key's row is read in 16-byte
//            pieces and meets the queries of all heads of the group (from LDS); the scaled scores, penalties taken
//            off, go to S [token][head][key] and the part's maximum and sum of exponentials per head to ml.
//   values   a workgroup a (token, kv head, part): from ml every head's maximum and sum over all parts (with its
//            sink); a thread a key forms the key's normalised weight for every head of the group, or, with a mixing
//            matrix, sum_g talk[h][g] w_g from the weights of all heads; then the threads, each a value channel and
//            a share of the part's pages, sum weight * value for the group's heads; partial sums per part go to po.
//   merge    out[token][head] = gate * sum over the parts that hold a visible key.
// Heads are taken sixteen at a time (or as many as the group has, rounded up to a power of two).  Layouts as above: K [page][kv head][offset][hd], V [page][kv head][vd][offset].
namespace {
constexpr int DEC_KEYS = 256;         // keys a part, threads a workgroup
constexpr int DEC_HEADS = 16;         // heads of a group taken together
constexpr int DEC_MAX_H = 256;

__device__ __forceinline__ float block_max_256(float v, float* scratch) {
    v = wave_max(v);
    __syncthreads();
    if (threadIdx.x % WAVE == 0) scratch[threadIdx.x / WAVE] = v;
    __syncthreads();
    return fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
}
__device__ __forceinline__ float block_sum_256(float v, float* scratch) {
    v = wave_sum(v);
    __syncthreads();
    if (threadIdx.x % WAVE == 0) scratch[threadIdx.x / WAVE] = v;
    __syncthreads();
    return (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
}

template <int GC>
__global__ __launch_bounds__(DEC_KEYS) void decode_scores_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, float* __restrict__ S, float* __restrict__ ml,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ req_of_token, const int* __restrict__ positions,
    int H, int Hkv, int hd, int page_size, int window, float scale, const float* __restrict__ slopes,
    const float* __restrict__ log_r1, const float* __restrict__ log_r2, int n_parts, int chunks) {
    __shared__ float qs[DEC_HEADS * 256];
    __shared__ float red_m[DEC_HEADS * 4], red_l[DEC_HEADS * 4];      // the four waves' maxima and sums of every head
    // (a group of more than GC heads is shared out among `chunks` workgroups, GC heads at a time each)
    const int t = blockIdx.x, kvh = blockIdx.y / chunks, chunk = blockIdx.y % chunks, part = blockIdx.z, tid = threadIdx.x;
    const int G = H / Hkv;
    const int pos = positions[blockIdx.x];
    const int lo = (window > 0) ? max(0, pos - window + 1) : 0;
    const int key = part * DEC_KEYS + tid;
    const bool part_live = part * DEC_KEYS <= pos && part * DEC_KEYS + DEC_KEYS - 1 >= lo;
    const bool valid = key >= lo && key <= pos;
    const bf16_t* krow = k_cache;
    if (valid) {
        const long long page = block_table[(long long)req_of_token[t] * max_blocks + key / page_size];
        krow = k_cache + ((page * Hkv + kvh) * page_size + key % page_size) * hd;
    }
    const float dist = (float)(pos - key);
    for (int g0 = chunk * GC; g0 < G; g0 += chunks * GC) {
        const int Gc = min(GC, G - g0);
        const int head0 = kvh * G + g0;
        if (!part_live) {                                       // uniform: no key of the part is visible
            if (tid < Gc) {
                float* dst = ml + (((long long)t * H + head0 + tid) * n_parts + part) * 2;
                dst[0] = -INFINITY;
                dst[1] = 0.f;
            }
            continue;
        }
        __syncthreads();
        for (int i = tid; i < Gc * hd; i += DEC_KEYS) qs[i] = to_f32(q[((long long)t * H + head0) * hd + i]);
        __syncthreads();
        float acc[GC];
#pragma unroll
        for (int g = 0; g < GC; ++g) acc[g] = 0.f;
        if (valid) {
            for (int c0 = 0; c0 < hd; c0 += 32) {            // four pieces of the row are loaded before any is used
                bf16x8 kv[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
                    kv[u] = c0 + 8 * u < hd ? *(const bf16x8*)(krow + c0 + 8 * u) : z;
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int c = c0 + 8 * u;
                    if (c >= hd) break;
                    float kf[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) kf[e] = (float)kv[u][e];
#pragma unroll
                    for (int g = 0; g < GC; ++g) {                  // (g >= Gc: whatever LDS holds, never stored)
                        const float* qg = qs + g * hd + c;
#pragma unroll
                        for (int e = 0; e < 8; ++e) acc[g] = fmaf(qg[e], kf[e], acc[g]);
                    }
                }
            }
        }
        // The part's maximum and sum of every head: the waves' own maxima (sums) of all heads first, then one exchange
        // through LDS for all of them, where a reduction a head at a time would cross the workgroup's barrier twice a
        // head.  The waves' values meet in the order of block_max_256 and block_sum_256: the same bits.
        float sv[GC], red[GC];
#pragma unroll
        for (int g = 0; g < GC; ++g) {
            const int head = head0 + min(g, Gc - 1);
            float s = -INFINITY;
            if (valid && g < Gc) {
                s = acc[g] * scale;
                if (slopes) s -= slopes[head] * dist;
                if (log_r1) s -= log_r1[head] * log1pf(log_r2[head] * dist);
                S[((long long)t * H + head) * n_parts * DEC_KEYS + key] = s;
            }
            sv[g] = s;
            red[g] = wave_max(s);
        }
        __syncthreads();                                        // (everybody has read qs; red_m and red_l are free)
        if (tid % WAVE == 0) {
#pragma unroll
            for (int g = 0; g < GC; ++g) red_m[g * 4 + tid / WAVE] = red[g];
        }
        __syncthreads();
        float m[GC];
#pragma unroll
        for (int g = 0; g < GC; ++g) {
            m[g] = fmaxf(fmaxf(red_m[g * 4], red_m[g * 4 + 1]), fmaxf(red_m[g * 4 + 2], red_m[g * 4 + 3]));
            red[g] = wave_sum((valid && g < Gc) ? expf(sv[g] - m[g]) : 0.f);
        }
        if (tid % WAVE == 0) {
#pragma unroll
            for (int g = 0; g < GC; ++g) red_l[g * 4 + tid / WAVE] = red[g];
        }
        __syncthreads();
        if (tid < Gc) {
            float* dst = ml + (((long long)t * H + head0 + tid) * n_parts + part) * 2;
            dst[0] = fmaxf(fmaxf(red_m[tid * 4], red_m[tid * 4 + 1]), fmaxf(red_m[tid * 4 + 2], red_m[tid * 4 + 3]));
            dst[1] = (red_l[tid * 4] + red_l[tid * 4 + 1]) + (red_l[tid * 4 + 2] + red_l[tid * 4 + 3]);
        }
    }
}

template <int GC>
__global__ __launch_bounds__(DEC_KEYS) void decode_values_kernel(
    const float* __restrict__ S, const float* __restrict__ ml, const bf16_t* __restrict__ v_cache, float* __restrict__ po,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ req_of_token, const int* __restrict__ positions,
    int H, int Hkv, int vd, int page_size, int window, const float* __restrict__ sinks, const float* __restrict__ talk, int n_parts,
    int chunks) {
    __shared__ float m_all[DEC_MAX_H], inv_all[DEC_MAX_H];
    __shared__ float w[DEC_HEADS * DEC_KEYS];                 // weights [head of the group][key]; then the slices' sums
    const int t = blockIdx.x, kvh = blockIdx.y / chunks, chunk = blockIdx.y % chunks, part = blockIdx.z, tid = threadIdx.x;
    const int g_first = chunk * GC;                           // the first heads of the group this workgroup takes
    const int G = H / Hkv;
    const int pos = positions[blockIdx.x];
    const int lo = (window > 0) ? max(0, pos - window + 1) : 0;
    if (part * DEC_KEYS > pos || part * DEC_KEYS + DEC_KEYS - 1 < lo) return;        // the merge skips such parts
    const int key = part * DEC_KEYS + tid;
    const bool valid = key >= lo && key <= pos;
    const int* table = block_table + (long long)req_of_token[t] * max_blocks;
    // What depends on nothing the kernel computes is asked for first, so that memory is waited for once: the part's page
    // numbers (into LDS), and without a mixing matrix the key's scores for the first heads of the group.
    __shared__ int page_of[DEC_KEYS / 8];
    if (tid < DEC_KEYS / page_size) {
        const int key0 = part * DEC_KEYS + tid * page_size;
        page_of[tid] = (key0 <= pos && key0 + page_size - 1 >= lo) ? table[key0 / page_size] : 0;
    }
    float s_first[GC];
#pragma unroll
    for (int g = 0; g < GC; ++g)
        s_first[g] = (!talk && valid && g_first + g < G) ? S[((long long)t * H + kvh * G + g_first + g) * n_parts * DEC_KEYS + key] : -INFINITY;
    // every head's maximum and sum over the parts (all heads with a mixing matrix, else the group's)
    const int h_first = talk ? 0 : kvh * G, h_count = talk ? H : G;
    // (eight lanes a head, each a share of the parts, so that the loads are in flight together)
    for (int i0 = 0; i0 < h_count; i0 += DEC_KEYS / 8) {
        const int i = i0 + tid / 8, sub = tid % 8;
        const bool live = i < h_count;
        const int head = h_first + (live ? i : 0);
        const float2* src = (const float2*)(ml + ((long long)t * H + head) * n_parts * 2);
        float M = -INFINITY, L = 0.f;
        for (int p = sub; p < n_parts; p += 8) {
            const float2 v = src[p];
            const float M2 = fmaxf(M, v.x);
            if (M2 > -INFINITY) L = L * expf(M - M2) + v.y * expf(v.x - M2);             // (a part without keys: -inf, 0)
            M = M2;
        }
#pragma unroll
        for (int off = 1; off < 8; off *= 2) {
            const float Mo = __shfl_xor(M, off, WAVE), Lo = __shfl_xor(L, off, WAVE);
            const float M2 = fmaxf(M, Mo);
            if (M2 > -INFINITY) L = L * expf(M - M2) + Lo * expf(Mo - M2);
            M = M2;
        }
        if (sinks) {
            const float sk = sinks[head], M2 = fmaxf(M, sk);
            L = L * expf(M - M2) + expf(sk - M2);
            M = M2;
        }
        if (live && sub == 0) {
            m_all[i] = M;
            inv_all[i] = 1.0f / L;
        }
    }
    const int slices = max(1, DEC_KEYS / vd);                   // threads (channel, slice of the part's pages)
    const int d = tid % vd, sl = tid / vd;
    const bool works = tid < vd * slices;
    for (int g0 = g_first; g0 < G; g0 += chunks * GC) {
        const int Gc = min(GC, G - g0);
        const int head0 = kvh * G + g0;
        __syncthreads();
        // ---- the key's weights
        float wk[GC];
#pragma unroll
        for (int g = 0; g < GC; ++g) wk[g] = 0.f;
        if (valid) {
            if (talk) {
                for (int h0 = 0; h0 < H; h0 += 8) {          // eight heads' scores are loaded before any is used
                    float sv[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u)
                        sv[u] = h0 + u < H ? S[((long long)t * H + h0 + u) * n_parts * DEC_KEYS + key] : -INFINITY;
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int h2 = h0 + u;
                        if (h2 >= H) break;
                        const float e = expf(sv[u] - m_all[h2]) * inv_all[h2];
#pragma unroll
                        for (int g = 0; g < GC; ++g) wk[g] = fmaf(talk[min(head0 + g, H - 1) * H + h2], e, wk[g]);
                    }
                }
            } else {
#pragma unroll
                for (int g = 0; g < GC; ++g)
                    if (g < Gc) {
                        const float sc = g0 == g_first ? s_first[g] : S[((long long)t * H + head0 + g) * n_parts * DEC_KEYS + key];
                        wk[g] = expf(sc - m_all[g0 + g]) * inv_all[g0 + g];
                    }
            }
        }
#pragma unroll
        for (int g = 0; g < GC; ++g)
            if (g < Gc) w[g * DEC_KEYS + tid] = wk[g];
        __syncthreads();
        // ---- weight * value
        float acc[GC];
#pragma unroll
        for (int g = 0; g < GC; ++g) acc[g] = 0.f;
        if (works) {
            // pieces of 8 keys; the page numbers and then the values of four pieces are loaded before any is used
            constexpr int PIECES = DEC_KEYS / 8;
            for (int c0 = sl; c0 < PIECES; c0 += 4 * slices) {
                const bf16_t* src[4];
                bool live[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int piece = c0 + u * slices;
                    const int key0 = part * DEC_KEYS + piece * 8;
                    live[u] = piece < PIECES && key0 <= pos && key0 + 7 >= lo;
                    const long long page = live[u] ? page_of[(piece * 8) / page_size] : 0;
                    src[u] = v_cache + ((page * Hkv + kvh) * vd + d) * page_size + key0 % page_size;
                }
                bf16x8 vv[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
                    vv[u] = live[u] ? *(const bf16x8*)src[u] : z;
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (!live[u]) continue;
                    const int piece = c0 + u * slices;
                    const int key0 = part * DEC_KEYS + piece * 8;
                    const float* wrow = w + piece * 8;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        // (positions after the last were never written: their weight is 0, but 0 * NaN is not)
                        const float vf = key0 + e <= pos ? (float)vv[u][e] : 0.f;
#pragma unroll
                        for (int g = 0; g < GC; ++g) acc[g] = fmaf(wrow[g * DEC_KEYS + e], vf, acc[g]);     // (g >= Gc: never stored)
                    }
                }
            }
        }
        __syncthreads();
        if (works && sl > 0) {
#pragma unroll
            for (int g = 0; g < GC; ++g)
                if (g < Gc) w[(g * slices + sl) * vd + d] = acc[g];
        }
        __syncthreads();
        if (works && sl == 0) {
#pragma unroll
            for (int g = 0; g < GC; ++g) {
                if (g < Gc) {
                    float sum = acc[g];
                    for (int s2 = 1; s2 < slices; ++s2) sum += w[(g * slices + s2) * vd + d];
                    po[(((long long)t * H + head0 + g) * n_parts + part) * vd + d] = sum;
                }
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(WAVE) void decode_merge_kernel(const float* __restrict__ po, const int* __restrict__ positions,
                                                            const float* __restrict__ gates, int gate_stride, T* __restrict__ out,
                                                            int H, int vd, int window, int n_parts) {
    const long long t = blockIdx.x;
    const int head = blockIdx.y;
    const int pos = positions[blockIdx.x];
    const int lo = (window > 0) ? max(0, pos - window + 1) : 0;
    const float g = gates ? 1.0f / (1.0f + expf(-gates[t * gate_stride + head])) : 1.f;
    for (int d = threadIdx.x; d < vd; d += WAVE) {
        float sum = 0.f;
        for (int p = 0; p < n_parts; ++p) {
            if (p * DEC_KEYS > pos || p * DEC_KEYS + DEC_KEYS - 1 < lo) continue;
            sum += po[((t * H + head) * n_parts + p) * vd + d];
        }
        out[(t * H + head) * vd + d] = from_f32<T>(sum * g);
    }
}
}  // namespace

// Single tokens, bfloat16 q and caches, float32 weights.  S float32 [tokens * H * n_parts * 256], ml float32
// [tokens * H * n_parts * 2] and po float32 [tokens * H * n_parts * vd] are work space; n_parts * 256 covers every position + 1.
// talk float32 [H][H] or null; gates float32 (row stride gate_stride) or null; out_dt: type of out [tokens][H][vd].
TUFF_EXPORT int tuff_attention_decode_exact(const void* q, const void* k_cache, const void* v_cache, void* out, int out_dt,
                                            float* S, float* ml, float* po, const int* block_table, int max_blocks,
                                            const int* req_of_token, const int* positions, int n_tokens, int H, int Hkv, int hd,
                                            int vd, int page_size, int window, float scale, const float* sinks, const float* slopes,
                                            const float* log_r1, const float* log_r2, const float* talk, const float* gates,
                                            int gate_stride, int n_parts, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (Hkv <= 0 || H % Hkv != 0 || H > DEC_MAX_H || hd % 8 != 0 || hd > 256 || vd <= 0 || vd > DEC_KEYS) return -2;
    if (page_size % 8 != 0 || DEC_KEYS % page_size != 0 || n_parts <= 0 || n_parts > 65535 || Hkv > 65535) return -2;
    if ((log_r1 == nullptr) != (log_r2 == nullptr) || !S || !ml || !po) return -2;
    // a group of more than sixteen heads (one row a position for every head, as latent attention has) is shared out
    // among several workgroups, sixteen heads each: the keys and values come from the caches once more, the step's few
    // workgroups become as many more
    const int chunks = (H / Hkv + DEC_HEADS - 1) / DEC_HEADS;
    if ((long long)Hkv * chunks > 65535) return -2;
    dim3 grid(n_tokens, Hkv * chunks, n_parts), block(DEC_KEYS);
    // (the loops over a group's heads are unrolled to the power of two that holds them, sixteen at most)
#define LAUNCH(GC) do { \
    hipLaunchKernelGGL(decode_scores_kernel<GC>, grid, block, 0, stream, (const bf16_t*)q, (const bf16_t*)k_cache, S, ml, block_table, \
                       max_blocks, req_of_token, positions, H, Hkv, hd, page_size, window, scale, slopes, log_r1, log_r2, n_parts, chunks); \
    hipLaunchKernelGGL(decode_values_kernel<GC>, grid, block, 0, stream, (const float*)S, (const float*)ml, (const bf16_t*)v_cache, po, \
                       block_table, max_blocks, req_of_token, positions, H, Hkv, vd, page_size, window, sinks, talk, n_parts, chunks); } while (0)
    const int G = H / Hkv;
    if (G <= 1) LAUNCH(1); else if (G <= 2) LAUNCH(2); else if (G <= 4) LAUNCH(4); else if (G <= 8) LAUNCH(8); else LAUNCH(16);
#undef LAUNCH
    dim3 mgrid(n_tokens, H), mblock(WAVE);
    if (out_dt == DT_F32)
        hipLaunchKernelGGL(decode_merge_kernel<float>, mgrid, mblock, 0, stream, (const float*)po, positions, gates, gate_stride,
                           (float*)out, H, vd, window, n_parts);
    else
        hipLaunchKernelGGL(decode_merge_kernel<bf16_t>, mgrid, mblock, 0, stream, (const float*)po, positions, gates, gate_stride,
                           (bf16_t*)out, H, vd, window, n_parts);
    return launch_status();
}
