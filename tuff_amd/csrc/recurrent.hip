// Kernels of mixers that carry a fixed-size state from token to token: the blend of a token's input
// with the one before it (token shift), a short causal convolution per channel with an activation,
// and four matrix-state recurrences, a decaying outer-product memory with a bonus for the current
// token ("wkv"), a gated delta rule (a decay per key channel or one per head), a memory whose forget gate also
// sets the write strength, and the state-space recurrence with a scalar decay per head ("ssd").  States are float32 and live in a slot per request; a step
// brings each request's next tokens (one decoded token or a portion of a prompt of any length),
// tokens flat and ordered by request, and every kernel continues from the slot and leaves it ready
// for the next step.  The recurrences run token by token in one fixed order of operations, so a
// position's result does not depend on how the sequence was cut into steps.
//
// Everything that enters a recurrence besides the projected rows is float32: decays, their
// exponentials and softplus, the write strength, the unit norms of q and k.
//
// Requests with no tokens in the step (q_len 0: a recorded step's padding) are skipped everywhere.
#include "common.h"
#include <math.h>

namespace {

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float siluf_(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// ------------------------------------------------------------------------ token shift
// out[s][t][c] = h[t][c] + (prev - h[t][c]) * mu[s][c], prev = the request's token before (its
// state where t is the first of the step).  With q_len the workgroup of a request's first token, the only
// one that reads the request's state, also leaves the state for the next step, the request's last row of
// this step (each thread after its own read of the same place): no second kernel.
template <typename T>
__global__ void shift_mix_kernel(const T* __restrict__ h, float* __restrict__ prev_state, const float* __restrict__ mu,
                                 T* __restrict__ out, const int* __restrict__ req_of_token, const int* __restrict__ q_start,
                                 const int* __restrict__ q_len, const int* __restrict__ state_slot, int n_tokens, int d, int n_mix) {
    const int t = blockIdx.x;
    const int r = req_of_token[t];
    const bool first = t == q_start[r];
    float* ps = prev_state + (long long)state_slot[r] * d;
    const T* hp = h + (long long)(t - 1) * d;
    const T* hc = h + (long long)t * d;
    const T* hl = (first && q_len) ? h + (long long)(t + q_len[r] - 1) * d : nullptr;
    for (int c = threadIdx.x; c < d; c += blockDim.x) {
        const float x = to_f32(hc[c]);
        const float p = first ? ps[c] : to_f32(hp[c]);
        for (int s = 0; s < n_mix; ++s)
            out[((long long)s * n_tokens + t) * d + c] = from_f32<T>(fmaf(p - x, mu[(long long)s * d + c], x));
        if (hl) ps[c] = to_f32(hl[c]);
    }
}

// prev_state[slot] = the request's last row of the step
template <typename T>
__global__ void shift_state_kernel(const T* __restrict__ h, float* __restrict__ prev_state, const int* __restrict__ q_start,
                                   const int* __restrict__ q_len, const int* __restrict__ state_slot, int d) {
    const int r = blockIdx.x;
    const int n = q_len[r];
    if (n <= 0) return;
    const T* src = h + (long long)(q_start[r] + n - 1) * d;
    float* dst = prev_state + (long long)state_slot[r] * d;
    for (int c = threadIdx.x; c < d; c += blockDim.x) dst[c] = to_f32(src[c]);
}

// --------------------------------------------------------------- short causal convolution
// y[t][c] = act(sum_j taps[c][j] x[t - (K-1) + j][c] + bias[c]); inputs before the step's first token come from
// the request's state [K-1][C] (zeros for a new request).  act: 0 none, 1 silu.  The rows of x lie ldx elements
// apart (they may be a column range of a wider projected row) and may be of another type than y's.
constexpr int MAX_TAPS = 17;

template <typename T, typename TY>
__global__ void conv_act_kernel(const T* __restrict__ x, long long ldx, const float* __restrict__ taps, const float* __restrict__ bias,
                                const float* __restrict__ state, TY* __restrict__ y, const int* __restrict__ req_of_token,
                                const int* __restrict__ q_start, const int* __restrict__ state_slot, int C, int K, int act) {
    const int t = blockIdx.x;
    const int r = req_of_token[t];
    const int i = t - q_start[r];                     // index within the step's portion
    const float* st = state + (long long)state_slot[r] * (K - 1) * C;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
        float acc = bias ? bias[c] : 0.f;
        for (int j = 0; j < K; ++j) {
            const int li = i - (K - 1) + j;
            const float v = li >= 0 ? to_f32(x[(long long)(t - (K - 1) + j) * ldx + c]) : st[(long long)(i + j) * C + c];
            acc = fmaf(taps[(long long)c * K + j], v, acc);
        }
        y[(long long)t * C + c] = from_f32<TY>(act == 1 ? siluf_(acc) : acc);
    }
}

// the state after the step: the last K-1 inputs, from the step's rows and, for a short portion, the old state
template <typename T>
__global__ void conv_state_kernel(const T* __restrict__ x, long long ldx, float* __restrict__ state, const int* __restrict__ q_start,
                                  const int* __restrict__ q_len, const int* __restrict__ state_slot, int C, int K) {
    const int r = blockIdx.x;
    const int n = q_len[r];
    if (n <= 0) return;
    float* st = state + (long long)state_slot[r] * (K - 1) * C;
    const int t0 = q_start[r];
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
        float keep[MAX_TAPS - 1];
#pragma unroll
        for (int m = 0; m < MAX_TAPS - 1; ++m) {
            if (m < K - 1) {
                const int li = n - (K - 1) + m;
                keep[m] = li >= 0 ? to_f32(x[(long long)(t0 + li) * ldx + c]) : st[(long long)(m + n) * C + c];
            }
        }
#pragma unroll
        for (int m = 0; m < MAX_TAPS - 1; ++m)
            if (m < K - 1) st[(long long)m * C + c] = keep[m];
    }
}

// ------------------------------------------------------------------------ recurrences
// Two kernels.  The first works on all tokens at once, a wave a (token, head): what enters the recurrence
// besides the projected rows is made there in float32, the decay w = exp(-exp(lw + w0)) and the bonus
// sum_i r_i u_i k_i (wkv), or the decay g = exp(-exp(A_log) softplus(a + dt_bias)), the write strength
// sigmoid(b) and q and k as unit vectors per head (x / sqrt(sum x^2 + 1e-6), q also times D^-1/2) (delta).
//
// The second walks each request's tokens in order, one wave per (request, head, a few value channels).  SPLIT
// neighbouring lanes (4 for key sizes up to 32, else 16) share a value channel j and keep a share of the state's
// column S[0..D-1][j] each in registers (RP rows); their partial sums meet in exchanges inside the group, always
// in the same order.  A token is a chain of dependent steps for a wave, so what a wave does for a token is kept
// short and the head's columns are spread over many waves.
// Eight tokens at a time: what they bring for the key channels is fetched while the eight before are computed
// and staged through LDS, from where every lane reads it as broadcasts.  The arithmetic of a token is the same
// whatever the step holds, so the result does not depend on how a sequence was cut.
//
// wkv:    o_j = sum_i r_i S_ij + bonus v_j;   S_ij <- w_i S_ij + k_i v_j
// delta:  S_ij <- g_i S_ij;  e_j = beta (v_j - sum_i k_i S_ij);  S_ij <- S_ij + k_i e_j;  o_j = sum_i q_i S_ij
// forget: S_ij <- f_i S_ij + (1 - f_i) v_j;  o_j = sum_i q_i S_ij      (the read sees the token's own write; no key)
struct PrepArgs {
    const void *a, *k;              // r or q, k: rows of Ha*D of the compute type, lda apart
    float* decay;                   // in: lw or a [T][H*D]; out, in place: w or g
    const float* decay_bias;        // [H*D]: w0 or dt_bias
    const float* per_head;          // wkv: u [H][D];  delta: A_log [H]
    const float* beta_in;           // delta: b, a token's H values ld_small apart
    const float* head_decay_in;     // delta with one decay per head: a, a token's H values ld_small apart (decay_bias is
                                    // then [H]); null: the decay's inputs are a value per key channel, in `decay`
    long long ld_small;
    float *qn, *kn;                 // delta, out: unit vectors [T][H][D]
    float* scalar;                  // out [T][H]: bonus (wkv) or beta (delta)
    int H, Ha, D;
    long long lda;                  // elements between two tokens' rows of a and k
};

template <typename T, bool DELTA>
__global__ __launch_bounds__(WAVE) void scan_prep_kernel(PrepArgs p) {
    const long long t = blockIdx.x;
    const int head = blockIdx.y, lane = threadIdx.x;
    const int D = p.D, H = p.H, Ha = p.Ha;
    const int ha = head / (H / Ha);
    const T* pa = (const T*)p.a + t * p.lda + ha * D;
    const T* pk = (const T*)p.k + t * p.lda + ha * D;
    float* dec = p.decay + (t * H + head) * D;
    if (DELTA) {
        float qq = 0.f, kk = 0.f;
        for (int i = lane; i < D; i += WAVE) {
            const float q = to_f32(pa[i]), k = to_f32(pk[i]);
            qq = fmaf(q, q, qq);
            kk = fmaf(k, k, kk);
        }
        qq = wave_sum(qq); kk = wave_sum(kk);
        const float qn = (1.0f / sqrtf((float)D)) / sqrtf(qq + 1e-6f), kn = 1.0f / sqrtf(kk + 1e-6f);
        const float neg_rate = -expf(p.per_head[head]);
        const float g_head = p.head_decay_in
            ? expf(neg_rate * softplusf_(p.head_decay_in[t * p.ld_small + head] + p.decay_bias[head])) : 0.f;
        for (int i = lane; i < D; i += WAVE) {
            p.qn[(t * H + head) * D + i] = to_f32(pa[i]) * qn;
            p.kn[(t * H + head) * D + i] = to_f32(pk[i]) * kn;
            dec[i] = p.head_decay_in ? g_head : expf(neg_rate * softplusf_(dec[i] + p.decay_bias[head * D + i]));
        }
        if (lane == 0) p.scalar[t * H + head] = sigmoidf_(p.beta_in[t * p.ld_small + head]);
    } else {
        float bonus = 0.f;
        for (int i = lane; i < D; i += WAVE) {
            bonus = fmaf(to_f32(pa[i]) * p.per_head[head * D + i], to_f32(pk[i]), bonus);
            dec[i] = expf(-expf(dec[i] + p.decay_bias[head * D + i]));
        }
        bonus = wave_sum(bonus);
        if (lane == 0) p.scalar[t * H + head] = bonus;
    }
}

// What enters the forget-gate recurrence: x holds a token's projected rows [q (H*D) | z (H*D) | ...], ld apart;
// qn = silu(q) and f = lower + (1 - lower) sigmoid(z + bias), both float32 [T][H*D].
template <typename T>
__global__ void forget_prep_kernel(const T* __restrict__ x, long long ld, const float* __restrict__ bias,
                                   const float* __restrict__ lower, float* __restrict__ qn, float* __restrict__ f, int HD) {
    const long long t = blockIdx.x;
    const T* row = x + t * ld;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < HD; c += gridDim.y * blockDim.x) {
        const float lo = lower[c];
        qn[t * HD + c] = siluf_(to_f32(row[c]));
        f[t * HD + c] = lo + (1.0f - lo) * sigmoidf_(to_f32(row[HD + c]) + (bias ? bias[c] : 0.f));
    }
}

// What enters the state-space recurrence besides the convolved rows, float32 [T][H] each: the step size
// dt = softplus(dt_raw + dt_bias_h) and the decay exp(-exp(A_log_h) dt), one number for all state channels of a head.
// dt_raw float32, a token's H values ld_dt apart.
// log_decay (or null): the decay's logarithm, -exp(A_log_h) dt, for the chunked form.
__global__ void ssd_prep_kernel(const float* __restrict__ dt_raw, long long ld_dt, const float* __restrict__ dt_bias,
                                const float* __restrict__ A_log, float* __restrict__ dt_out, float* __restrict__ decay,
                                float* __restrict__ log_decay, long long n, int H) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const long long t = i / H;
    const int head = (int)(i % H);
    const float dt = softplusf_(dt_raw[t * ld_dt + head] + dt_bias[head]);
    const float la = -expf(A_log[head]) * dt;
    dt_out[i] = dt;
    decay[i] = expf(la);
    if (log_decay) log_decay[i] = la;
}

// ------------------------------------------------- the state-space recurrence in chunks, on the matrix cores
// For prompt portions in bfloat16 runs.  A request's tokens of the step are cut into chunks of 64 from the portion's
// first token.  With a_t the running sum of the decays' logarithms inside a chunk (a_t <= 0, falling), K_s = dt_s B_s and
// S_in the state at the chunk's start:
//     y_t = sum_{s <= t} exp(a_t - a_s) (C_t . K_s) x_s  +  exp(a_t) C_t^T S_in  +  D x_t
//     S_out = exp(a_last) S_in + sum_s exp(a_last - a_s) K_s x_s^T
// Three kernels: (1) every chunk's own contribution U = sum_s exp(a_last - a_s) K_s x_s^T and its decay exp(a_last), all
// chunks at once; (2) per request and head the chunks in order, an element of the state a thread: S_in of every chunk
// takes U's place, the last S_out goes to the slot; (3) every chunk's outputs, all chunks at once.  All factors, sums and
// the state are float32; the products run as float32 matrix instructions (16 x 16 x 4), whose operands are the float32
// values themselves (B, C and x are bfloat16 as the convolution left them, converted exactly).  Every exponent is <= 0.
// The sums of a token are formed in another order than token by token, so a position's result depends on where its
// portion began, within float32 rounding; a float32 run keeps the token-by-token kernel.
constexpr int CHUNK = 64;

__device__ __forceinline__ f32x4 mfma_f32(float a, float b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }

struct SsdChunkArgs {
    const bf16_t* xbc;              // a token's rows [x (H*P) | B (G*N) | C (G*N)], ld apart
    long long ld;
    const float *dt, *la;           // [T][H]: step size, logarithm of the decay
    const float* Dh;                // [H]
    float* state;                   // [slots][H][N][P]
    float* U;                       // [chunks][H][N][P]: a chunk's contribution, then the state at its start
    float* cdec;                    // [chunks][H]: exp(a_last)
    float* out;                     // [T][H][P]
    const int *q_start, *q_len, *state_slot;
    int R, H, G, N, P;
};

// Which request and which of its chunks workgroup `ci` takes (chunks are numbered request after request); false: none.
__device__ __forceinline__ bool chunk_of(const SsdChunkArgs& p, int ci, int& r, int& t0, int& L) {
    for (r = 0; r < p.R; ++r) {
        const int n = p.q_len[r];
        const int nc = (n + CHUNK - 1) / CHUNK;
        if (ci < nc) {
            t0 = p.q_start[r] + ci * CHUNK;
            L = min(CHUNK, n - ci * CHUNK);
            return true;
        }
        ci -= nc;
    }
    return false;
}

// a[t] = sum_{s <= t} la[s] over the chunk's tokens, by the first wave; sa[CHUNK] in LDS (a[t] = a[L-1] beyond the chunk)
__device__ __forceinline__ void chunk_prefix(const SsdChunkArgs& p, int t0, int L, int head, float* sa) {
    if (threadIdx.x < WAVE) {
        const int lane = threadIdx.x;
        float v = lane < L ? p.la[(long long)(t0 + lane) * p.H + head] : 0.f;
#pragma unroll
        for (int off = 1; off < WAVE; off *= 2) {
            const float up = __shfl_up(v, off, WAVE);
            if (lane >= off) v += up;
        }
        sa[lane] = v;
    }
}

// A lane's operands of consecutive matrix instructions lie side by side in LDS: the inner index of a product may be
// taken in any order as long as both operands agree, so lane group q (of four) takes the q-th quarter of it, and its
// operands of four instructions are one 16-byte (float32) or 8-byte (bfloat16) read.
__global__ __launch_bounds__(256) void ssd_chunk_state_kernel(SsdChunkArgs p) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    const int N = p.N, P = p.P, head = blockIdx.y, tid = threadIdx.x;
    int r, t0, L;
    if (!chunk_of(p, blockIdx.x, r, t0, L)) return;
    constexpr int LDS_ = CHUNK + 4;
    float* sa = sm;                               // [CHUNK]
    float* sw = sa + CHUNK;                       // [CHUNK]: exp(a_last - a_s) dt_s
    float* sBt = sw + CHUNK;                      // [N][CHUNK + 4]: w_s B_s[n], a state channel's tokens side by side
    float* sXt = sBt + N * LDS_;                  // [P][CHUNK + 4]
    chunk_prefix(p, t0, L, head, sa);
    __syncthreads();
    if (tid < CHUNK) sw[tid] = tid < L ? expf(sa[L - 1] - sa[tid]) * p.dt[(long long)(t0 + tid) * p.H + head] : 0.f;
    __syncthreads();
    const int g = head / (p.H / p.G);
    const bf16_t* base = p.xbc + (long long)t0 * p.ld;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const int NC = N / 8, PC = P / 8;
    for (int i = tid; i < CHUNK * NC; i += 256) {
        const int s_ = i / NC, ch = i % NC;
        const bf16x8 v = s_ < L ? *(const bf16x8*)(base + (long long)s_ * p.ld + (long long)p.H * P + (long long)g * N + ch * 8) : zero8;
        const float w = sw[s_];
#pragma unroll
        for (int e = 0; e < 8; ++e) sBt[(ch * 8 + e) * LDS_ + s_] = w * (float)v[e];
    }
    for (int i = tid; i < CHUNK * PC; i += 256) {
        const int s_ = i / PC, ch = i % PC;
        const bf16x8 v = s_ < L ? *(const bf16x8*)(base + (long long)s_ * p.ld + (long long)head * P + ch * 8) : zero8;
#pragma unroll
        for (int e = 0; e < 8; ++e) sXt[(ch * 8 + e) * LDS_ + s_] = (float)v[e];
    }
    __syncthreads();
    const int wave = tid / WAVE, lane = tid % WAVE, l16 = lane % 16, lq = lane / 16;
    const int NT = N / 16, PT = P / 16;
    float* U = p.U + ((long long)blockIdx.x * p.H + head) * N * P;
    for (int tile = wave; tile < NT * PT; tile += 4) {
        const int nt = tile / PT, pt = tile % PT;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        const float* pa = sBt + (nt * 16 + l16) * LDS_ + lq * (CHUNK / 4);
        const float* pb = sXt + (pt * 16 + l16) * LDS_ + lq * (CHUNK / 4);
#pragma unroll
        for (int j4 = 0; j4 < CHUNK / 16; ++j4) {
            const f32x4 a4 = *(const f32x4*)(pa + 4 * j4), b4 = *(const f32x4*)(pb + 4 * j4);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc = mfma_f32(a4[e], b4[e], acc);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) U[(long long)(nt * 16 + 4 * lq + e) * P + pt * 16 + l16] = acc[e];
    }
    if (tid == 0) p.cdec[(long long)blockIdx.x * p.H + head] = expf(sa[L - 1]);
}

__global__ __launch_bounds__(256) void ssd_state_pass_kernel(SsdChunkArgs p) {
    const int r = blockIdx.x, head = blockIdx.y;
    const int n = p.q_len[r];
    if (n <= 0) return;
    const long long NP = (long long)p.N * p.P;
    const long long e = (long long)blockIdx.z * 256 + threadIdx.x;
    if (e >= NP) return;
    int first = 0;
    for (int r2 = 0; r2 < r; ++r2) first += (p.q_len[r2] + CHUNK - 1) / CHUNK;
    const int nc = (n + CHUNK - 1) / CHUNK;
    float* S = p.state + ((long long)p.state_slot[r] * p.H + head) * NP + e;
    float s_ = *S;
    for (int c = 0; c < nc; ++c) {
        float* u = p.U + ((long long)(first + c) * p.H + head) * NP + e;
        const float own = *u;
        *u = s_;
        s_ = fmaf(p.cdec[(long long)(first + c) * p.H + head], s_, own);
    }
    *S = s_;
}

__global__ __launch_bounds__(256) void ssd_chunk_out_kernel(SsdChunkArgs p) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    const int N = p.N, P = p.P, head = blockIdx.y, tid = threadIdx.x;
    int r, t0, L;
    if (!chunk_of(p, blockIdx.x, r, t0, L)) return;
    constexpr int LDG = CHUNK + 4, LDXT = CHUNK + 8;
    const int ldn = N + 8;
    float* sa = sm;                               // [CHUNK]
    float* sdt = sa + CHUNK;                      // [CHUNK]
    float* sGt = sdt + CHUNK;                     // [CHUNK (t)][CHUNK + 4 (s)]: the masked, scaled C_t . B_s
    bf16_t* sB = (bf16_t*)(sGt + CHUNK * LDG);    // [CHUNK][N + 8]
    bf16_t* sC = sB + CHUNK * ldn;                // [CHUNK][N + 8]
    bf16_t* sXt = sC + CHUNK * ldn;               // [P][CHUNK + 8]: a channel's tokens side by side
    chunk_prefix(p, t0, L, head, sa);
    if (tid >= 64 && tid < 128) sdt[tid - 64] = tid - 64 < L ? p.dt[(long long)(t0 + tid - 64) * p.H + head] : 0.f;
    const int g = head / (p.H / p.G);
    const bf16_t* base = p.xbc + (long long)t0 * p.ld;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const int NC = N / 8, PC = P / 8;
    for (int i = tid; i < CHUNK * NC; i += 256) {
        const int s_ = i / NC, ch = i % NC;
        const bf16_t* row = base + (long long)s_ * p.ld + (long long)p.H * P + (long long)g * N + ch * 8;
        *(bf16x8*)(sB + s_ * ldn + ch * 8) = s_ < L ? *(const bf16x8*)row : zero8;
        *(bf16x8*)(sC + s_ * ldn + ch * 8) = s_ < L ? *(const bf16x8*)(row + (long long)p.G * N) : zero8;
    }
    for (int i = tid; i < CHUNK * PC; i += 256) {
        const int s_ = i / PC, ch = i % PC;
        const bf16x8 v = s_ < L ? *(const bf16x8*)(base + (long long)s_ * p.ld + (long long)head * P + ch * 8) : zero8;
#pragma unroll
        for (int e = 0; e < 8; ++e) sXt[(ch * 8 + e) * LDXT + s_] = v[e];
    }
    __syncthreads();
    const int wave = tid / WAVE, lane = tid % WAVE, l16 = lane % 16, lq = lane / 16;
    const int nq = N / 4;                          // a lane group's share of the state channels
    // Gt[t][s] = (s <= t) exp(a_t - a_s) dt_s sum_n B[s][n] C[t][n]; tiles above the diagonal are zero
    for (int tile = wave; tile < 16; tile += 4) {
        const int st = tile / 4, tt = tile % 4;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        if (st <= tt && st * 16 < L) {
            const bf16_t* pa = sB + (st * 16 + l16) * ldn + lq * nq;
            const bf16_t* pb = sC + (tt * 16 + l16) * ldn + lq * nq;
#pragma unroll 4
            for (int j4 = 0; j4 < nq / 4; ++j4) {
                const bf16x4 a4 = *(const bf16x4*)(pa + 4 * j4), b4 = *(const bf16x4*)(pb + 4 * j4);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc = mfma_f32((float)a4[e], (float)b4[e], acc);
            }
        }
        const int t = tt * 16 + l16;
        f32x4 gv;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int s_ = st * 16 + 4 * lq + e;
            gv[e] = (s_ <= t && t < L) ? acc[e] * expf(sa[t] - sa[s_]) * sdt[s_] : 0.f;
        }
        *(f32x4*)(sGt + t * LDG + st * 16 + 4 * lq) = gv;
    }
    __syncthreads();
    // y[t][c] = sum_s Gt[t][s] x[s][c] + exp(a_t) sum_n C[t][n] S_in[n][c] + D x[t][c]
    const float* Sin = p.U + ((long long)blockIdx.x * p.H + head) * N * P;
    const float dh = p.Dh[head];
    const int PT = P / 16;
    // a wave takes a block of 16 channels and walks the chunk's four blocks of tokens with it: its share of S_in's
    // columns (a lane group's quarter of the state channels, at most 32 numbers a lane) is read once, into registers
    for (int pt = wave; pt < PT; pt += 4) {
        const float* ps = Sin + (long long)(lq * nq) * P + pt * 16 + l16;
        float sreg[32];
#pragma unroll
        for (int k = 0; k < 32; ++k) sreg[k] = k < nq ? ps[(long long)k * P] : 0.f;
        const bf16_t* px = sXt + (pt * 16 + l16) * LDXT;
        for (int tt = 0; tt < 4; ++tt) {
            if (tt * 16 >= L) break;
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            const int sq = 4 * (tt + 1);           // a lane group's share of the keys up to the block's last row
            const float* pg = sGt + (tt * 16 + l16) * LDG + lq * sq;
            for (int j4 = 0; j4 <= tt; ++j4) {
                const f32x4 a4 = *(const f32x4*)(pg + 4 * j4);
                const bf16x4 b4 = *(const bf16x4*)(px + lq * sq + 4 * j4);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc = mfma_f32(a4[e], (float)b4[e], acc);
            }
            const float ea = expf(sa[min(tt * 16 + l16, L - 1)]);
            const bf16_t* pc = sC + (tt * 16 + l16) * ldn + lq * nq;
#pragma unroll
            for (int j4 = 0; j4 < 8; ++j4) {
                if (4 * j4 < nq) {
                    const bf16x4 c4 = *(const bf16x4*)(pc + 4 * j4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc = mfma_f32(ea * (float)c4[e], sreg[4 * j4 + e], acc);
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int t = tt * 16 + 4 * lq + e, c = pt * 16 + l16;
                if (t < L) p.out[((long long)(t0 + t) * p.H + head) * P + c] = fmaf(dh, (float)sXt[c * LDXT + t], acc[e]);
            }
        }
    }
}

struct ScanArgs {
    const void *a, *k, *v;          // per token: a (r, or unit q) and k, rows of Ha*D, lda apart; v: rows of H*Dv, ldv apart   (Ha: heads of a and k)
    const float* decay;             // per token [T][H*D]: w or g; ssd: [T][H], one decay for all of a head's key channels
    const float* scalar;            // per token [T][H]: bonus or beta; ssd: the step size dt, which multiplies the key
    float* state;                   // [slots][H][D][Dv]
    float* out;                     // [T][H][Dv]
    const int *q_start, *q_len, *state_slot;
    int H, Ha, D, Dv;
    long long ldv;                  // elements between two tokens' rows of v
    long long lda;                  // elements between two tokens' rows of a and k
    const float* head_bonus;        // ssd: [H], the factor of the token's own value in its output
};

constexpr int SCAN_CH = 8;          // tokens staged at a time

// The sum over the SPLIT neighbouring lanes that share a value channel, the same in all of them: exchanges
// inside a quad (lane ^ 1, then lane ^ 2) and, for 16, rotations by 4 and by 8 within the row of 16 lanes.
template <int CTRL>
__device__ __forceinline__ float dpp_of(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int SPLIT>
__device__ __forceinline__ float group_sum(float v) {
    v += dpp_of<0xB1>(v);
    v += dpp_of<0x4E>(v);
    if (SPLIT == 16) {
        v += dpp_of<0x124>(v);
        v += dpp_of<0x128>(v);
    }
    return v;
}

// TA: type of a and k (the compute type for wkv's r and k, float for the delta rule's unit vectors); T: type of v.
// FORGET: a holds silu(q) in float32, the decay is the forget gate f and the key is 1 - f (k and scalar are not used).
// SSD: S_ij <- w S_ij + (dt k_i) v_j with one decay w for the head, then o_j = sum_i a_i S_ij + bonus_h v_j (the read sees
// the token's own write); a and k are the convolved rows themselves (C and B of the head's group), of the compute type.
template <typename TA, typename T, int NI16, int SPLIT, bool DELTA, bool FORGET = false, bool SSD = false>
__global__ __launch_bounds__(WAVE) void scan_kernel(ScanArgs p) {
    constexpr int RP = NI16 * 4;                       // rows of the state's column a lane keeps
    constexpr int DP = RP * SPLIT;                     // key channels, padded
    constexpr int SCAN_COLS = WAVE / SPLIT;            // value channels a wave
    constexpr int PER = (DP + WAVE - 1) / WAVE;        // key channels a lane stages
    constexpr int CH = SCAN_CH;
    __shared__ __attribute__((aligned(16))) float sa[CH][DP];
    __shared__ __attribute__((aligned(16))) float sk[CH][DP];
    __shared__ __attribute__((aligned(16))) float sw[CH][DP];
    const int r = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int n = p.q_len[r];
    if (n <= 0) return;
    const int D = p.D, Dv = p.Dv, H = p.H, Ha = p.Ha;
    const int ha = head / (H / Ha);
    const int part = lane % SPLIT;
    const int j = blockIdx.z * SCAN_COLS + lane / SPLIT;
    const bool jv = j < Dv;
    const int row0 = part * RP;
    const int t0 = p.q_start[r];
    float* S = p.state + (((long long)p.state_slot[r] * H + head) * D) * Dv + j;
    const TA* pa = (const TA*)p.a;
    const TA* pk = (const TA*)p.k;
    const T* pv = (const T*)p.v;

    float s[RP];
#pragma unroll
    for (int i = 0; i < RP; ++i) s[i] = (jv && row0 + i < D) ? S[(long long)(row0 + i) * Dv] : 0.f;

    // what the next eight tokens bring
    // (kept as they were loaded: a conversion on the spot would wait for the load)
    TA fa[CH][PER], fk[CH][PER];
    T fv[CH];
    float fw[CH][PER], fb[CH];
    // Every load is issued whatever the lane and token (from a clamped place where there is nothing to fetch);
    // what does not count is replaced when the values are staged, eight tokens later: a load inside a condition
    // would be waited for on the spot, and so would a value that is looked at right after its load.
    // Addresses are a base that is the same for the whole wave (the chunk's first token, this head) plus a small
    // offset a lane: the rows of a chunk lie less than 2^31 elements apart.
    const int jc = min(j, Dv - 1);
    const unsigned strideA = (unsigned)p.lda, strideW = (unsigned)(H * D), strideV = (unsigned)p.ldv, strideS = (unsigned)H;
    const float bonus_h = SSD ? p.head_bonus[head] : 0.f;
    float fd[CH];                                      // ssd: a token's decay
    int ic[PER];
#pragma unroll
    for (int e = 0; e < PER; ++e) ic[e] = min(lane + e * WAVE, D - 1);
    auto fetch = [&](int first, int count) {
        const TA* ba = pa + (long long)first * p.lda + (long long)ha * D;
        const TA* bk = pk + (long long)first * p.lda + (long long)ha * D;
        const float* bw = SSD ? p.decay + (long long)first * H + head : p.decay + ((long long)first * H + head) * D;
        const T* bv = pv + (long long)first * p.ldv + (long long)head * Dv;
        const float* bs = p.scalar + (long long)first * H + head;
#pragma unroll
        for (int tt = 0; tt < CH; ++tt) {
            const unsigned tc = (unsigned)min(tt, count - 1);
#pragma unroll
            for (int e = 0; e < PER; ++e) {
                fa[tt][e] = ba[tc * strideA + (unsigned)ic[e]];
                fk[tt][e] = bk[tc * strideA + (unsigned)ic[e]];
                if (!SSD) fw[tt][e] = bw[tc * strideW + (unsigned)ic[e]];
            }
            if (SSD) fd[tt] = bw[tc * strideS];
            fv[tt] = bv[tc * strideV + (unsigned)jc];
            fb[tt] = bs[tc * strideS];
        }
    };
    // one token: the state's rows of this lane move on and the token's output leaves.  Four partial sums a
    // lane (rows 0, 1, 2, 3 of every group of four), added in a fixed order, then the quad's exchange.
    auto token = [&](int tt, float vt, float sc, float wt, float* orow) {
        float o4[4] = {0.f, 0.f, 0.f, 0.f};
        if (DELTA) {
            float kv4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int g4 = 0; g4 < NI16; ++g4) {
                const f32x4 w4 = *(const f32x4*)&sw[tt][row0 + g4 * 4];
                const f32x4 k4 = *(const f32x4*)&sk[tt][row0 + g4 * 4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s[g4 * 4 + e] *= w4[e];
                    kv4[e] = fmaf(k4[e], s[g4 * 4 + e], kv4[e]);
                }
            }
            const float err = sc * (vt - group_sum<SPLIT>((kv4[0] + kv4[1]) + (kv4[2] + kv4[3])));
#pragma unroll
            for (int g4 = 0; g4 < NI16; ++g4) {
                const f32x4 k4 = *(const f32x4*)&sk[tt][row0 + g4 * 4];
                const f32x4 q4 = *(const f32x4*)&sa[tt][row0 + g4 * 4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s[g4 * 4 + e] = fmaf(k4[e], err, s[g4 * 4 + e]);
                    o4[e] = fmaf(q4[e], s[g4 * 4 + e], o4[e]);
                }
            }
        } else {
#pragma unroll
            for (int g4 = 0; g4 < NI16; ++g4) {
                const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
                const f32x4 w4 = SSD ? zero4 : *(const f32x4*)&sw[tt][row0 + g4 * 4];
                const f32x4 k4 = *(const f32x4*)&sk[tt][row0 + g4 * 4];
                const f32x4 r4 = *(const f32x4*)&sa[tt][row0 + g4 * 4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (SSD) {
                        s[g4 * 4 + e] = fmaf(wt, s[g4 * 4 + e], k4[e] * vt);
                        o4[e] = fmaf(r4[e], s[g4 * 4 + e], o4[e]);
                    } else if (FORGET) {
                        s[g4 * 4 + e] = fmaf(w4[e], s[g4 * 4 + e], k4[e] * vt);
                        o4[e] = fmaf(r4[e], s[g4 * 4 + e], o4[e]);
                    } else {
                        o4[e] = fmaf(r4[e], s[g4 * 4 + e], o4[e]);
                        s[g4 * 4 + e] = fmaf(w4[e], s[g4 * 4 + e], k4[e] * vt);
                    }
                }
            }
        }
        float o = group_sum<SPLIT>((o4[0] + o4[1]) + (o4[2] + o4[3]));
        if (SSD) o = fmaf(bonus_h, vt, o);
        else if (!DELTA && !FORGET) o = fmaf(sc, vt, o);
        // (the lanes of a group hold the same sum and write it to the same place: no lane is switched off for it)
        if (jv) orow[(unsigned)tt * (unsigned)(H * Dv)] = o;
    };

    fetch(t0, min(n, CH));
    for (int c0 = 0; c0 < n; c0 += CH) {
        const int count = min(CH, n - c0);
        float v[CH], sc[CH], wd[CH];
#pragma unroll
        for (int tt = 0; tt < CH; ++tt) {
            v[tt] = to_f32(fv[tt]);
            sc[tt] = fb[tt];
            wd[tt] = SSD ? fd[tt] : 0.f;
#pragma unroll
            for (int e = 0; e < PER; ++e) {
                const int i = lane + e * WAVE;
                const bool ok = i < D;                 // (tokens beyond the chunk's last are staged and never read)
                if (i < DP) {
                    sa[tt][i] = ok ? to_f32(fa[tt][e]) : 0.f;
                    sk[tt][i] = ok ? (FORGET ? 1.0f - fw[tt][e] : SSD ? fb[tt] * to_f32(fk[tt][e]) : to_f32(fk[tt][e])) : 0.f;
                    if (!SSD) sw[tt][i] = ok ? fw[tt][e] : 0.f;
                }
            }
        }
        if (c0 + CH < n) fetch(t0 + c0 + CH, min(CH, n - c0 - CH));
        // The workgroup is one wave and LDS serves a wave's accesses in order: nothing has to be waited for
        // between the writes above and the reads below, only the compiler must keep their order.  (A
        // __syncthreads() would also wait for the loads of the next eight tokens, which are meant to be under
        // way while these are computed.)
        __builtin_amdgcn_wave_barrier();
        float* orow = p.out + ((long long)(t0 + c0) * H + head) * Dv + j;     // this lane's place in the chunk's first row
        if (count == CH) {                             // eight whole tokens: no test between them
#pragma unroll
            for (int tt = 0; tt < CH; ++tt) token(tt, v[tt], sc[tt], wd[tt], orow);
        } else {
#pragma unroll
            for (int tt = 0; tt < CH; ++tt)
                if (tt < count) token(tt, v[tt], sc[tt], wd[tt], orow);
        }
        __builtin_amdgcn_wave_barrier();               // the reads stay before the next tokens' writes
    }
#pragma unroll
    for (int i = 0; i < RP; ++i)
        if (jv && row0 + i < D) S[(long long)(row0 + i) * Dv] = s[i];
}

// ---------------------------------------------------------- per-head unit norm, weight and gate
// y[t][h][j] = o[t][h][j] / sqrt(mean_j o^2 + eps) * w[(h * w_stride) + j] * f(gate[t][h][j]);
// f: 0 identity, 1 silu, 2 sigmoid; without a gate the factor is 1.  A wave per (token, head).
// gate_first: the gate comes before the norm, y = u / sqrt(mean_j u^2 + eps) * w with u = o f(gate).
// A token's gates lie gate_ld elements apart (they may be a column range of a wider projected row).
template <typename TG, typename T>
__global__ __launch_bounds__(WAVE) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w, int w_stride,
                                                              const TG* __restrict__ gate, long long gate_ld, int gate_fn, int gate_first,
                                                              T* __restrict__ y, int H, int Dv, float eps) {
    const long long row = (long long)blockIdx.x * H + blockIdx.y;
    const float* src = o + row * Dv;
    const TG* gr = gate ? gate + (long long)blockIdx.x * gate_ld + (long long)blockIdx.y * Dv : nullptr;
    auto gate_of = [&](int j) {
        float g = gr ? to_f32(gr[j]) : 1.f;
        if (gate_fn == 1) g = siluf_(g);
        else if (gate_fn == 2) g = sigmoidf_(g);
        return g;
    };
    float ss = 0.f;
    for (int j = threadIdx.x; j < Dv; j += WAVE) {
        const float u = gate_first ? src[j] * gate_of(j) : src[j];
        ss = fmaf(u, u, ss);
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)Dv + eps);
    for (int j = threadIdx.x; j < Dv; j += WAVE) {
        const float wj = w[(long long)blockIdx.y * w_stride + j];
        const float g = gate_of(j);
        y[row * Dv + j] = from_f32<T>(gate_first ? (src[j] * g) * inv * wj : src[j] * inv * wj * g);
    }
}

template <typename TA, typename T, bool DELTA, bool FORGET = false, bool SSD = false>
int launch_scan(const ScanArgs& p, int R, hipStream_t stream) {
    if (p.H > 65535 || p.D > 256) return -2;
    const bool narrow = p.D <= 32;                      // four lanes a value channel; else sixteen
    const int split = narrow ? 4 : 16;
    const int ni = narrow ? (p.D + 15) / 16 : (p.D + 63) / 64;
    dim3 grid(R, p.H, ceil_div(p.Dv, WAVE / split)), block(WAVE);
    if (grid.z > 65535) return -2;
#define SCAN(NI, SPLIT) hipLaunchKernelGGL((scan_kernel<TA, T, NI, SPLIT, DELTA, FORGET, SSD>), grid, block, 0, stream, p)
    if (narrow) { if (ni <= 1) SCAN(1, 4); else SCAN(2, 4); }
    else if (ni <= 1) SCAN(1, 16);
    else if (ni <= 2) SCAN(2, 16);
    else if (ni <= 3) SCAN(3, 16);
    else SCAN(4, 16);
#undef SCAN
    return launch_status();
}
}  // namespace

// q_len null: the state is only read.
TUFF_EXPORT int tuff_shift_mix(const void* h, int dt, float* prev_state, const float* mu, void* out,
                               const int* req_of_token, const int* q_start, const int* q_len, const int* state_slot,
                               int n_tokens, int d, int n_mix, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens), block(256);
    if (dt == DT_F32) hipLaunchKernelGGL(shift_mix_kernel<float>, grid, block, 0, stream, (const float*)h, prev_state, mu, (float*)out, req_of_token, q_start, q_len, state_slot, n_tokens, d, n_mix);
    else hipLaunchKernelGGL(shift_mix_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)h, prev_state, mu, (bf16_t*)out, req_of_token, q_start, q_len, state_slot, n_tokens, d, n_mix);
    return launch_status();
}

TUFF_EXPORT int tuff_shift_state(const void* h, int dt, float* prev_state, const int* q_start, const int* q_len,
                                 const int* state_slot, int n_requests, int d, hipStream_t stream) {
    if (n_requests <= 0) return 0;
    dim3 grid(n_requests), block(256);
    if (dt == DT_F32) hipLaunchKernelGGL(shift_state_kernel<float>, grid, block, 0, stream, (const float*)h, prev_state, q_start, q_len, state_slot, d);
    else hipLaunchKernelGGL(shift_state_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)h, prev_state, q_start, q_len, state_slot, d);
    return launch_status();
}

// x [T] rows of C channels ldx elements apart, of type dt; y [T][C] of type out_dt (where the types differ x is
// float32); taps float32 [C][K]; bias float32 [C] or null; state float32 [slots][K-1][C].  q_len null: the state is
// only read.
TUFF_EXPORT int tuff_conv_act(const void* x, int dt, long long ldx, const float* taps, const float* bias, float* state, void* y,
                              int out_dt, const int* req_of_token, const int* q_start, const int* q_len, const int* state_slot,
                              int n_tokens, int n_requests, int C, int K, int act, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (K < 1 || K > MAX_TAPS || ldx < C || (dt != out_dt && dt != DT_F32)) return -2;
    const int cols = ceil_div(C, 256);
    dim3 block(256);
#define CONV(T, TY) hipLaunchKernelGGL((conv_act_kernel<T, TY>), dim3(n_tokens, cols), block, 0, stream, (const T*)x, ldx, taps, bias, state, (TY*)y, req_of_token, q_start, state_slot, C, K, act)
    if (dt == DT_F32 && out_dt == DT_F32) CONV(float, float);
    else if (dt == DT_F32) CONV(float, bf16_t);
    else CONV(bf16_t, bf16_t);
#undef CONV
    int rc = launch_status();
    if (rc != 0 || !q_len || K == 1) return rc;
    if (dt == DT_F32) hipLaunchKernelGGL(conv_state_kernel<float>, dim3(n_requests, cols), block, 0, stream, (const float*)x, ldx, state, q_start, q_len, state_slot, C, K);
    else hipLaunchKernelGGL(conv_state_kernel<bf16_t>, dim3(n_requests, cols), block, 0, stream, (const bf16_t*)x, ldx, state, q_start, q_len, state_slot, C, K);
    return launch_status();
}

// wkv: r, k, v [T][H*D] of type dt; lw float32 [T][H*D] (overwritten with the decays); w0 float32 [H*D]; u float32
// [H][D]; bonus float32 [T][H] (work array); state float32 [slots][H][D][D]; out float32 [T][H][D].
TUFF_EXPORT int tuff_wkv_scan(const void* r, const void* k, const void* v, int dt, float* lw, const float* w0,
                              const float* u, float* bonus, float* state, float* out, const int* q_start, const int* q_len,
                              const int* state_slot, int n_tokens, int n_requests, int H, int D, hipStream_t stream) {
    if (n_requests <= 0 || n_tokens <= 0) return 0;
    if (H > 65535) return -2;
    PrepArgs pp{r, k, lw, w0, u, nullptr, nullptr, 0, nullptr, nullptr, bonus, H, H, D, (long long)H * D};
    if (dt == DT_F32) hipLaunchKernelGGL((scan_prep_kernel<float, false>), dim3(n_tokens, H), dim3(WAVE), 0, stream, pp);
    else hipLaunchKernelGGL((scan_prep_kernel<bf16_t, false>), dim3(n_tokens, H), dim3(WAVE), 0, stream, pp);
    ScanArgs p{r, k, v, lw, bonus, state, out, q_start, q_len, state_slot, H, H, D, D, (long long)H * D, (long long)H * D, nullptr};
    return dt == DT_F32 ? launch_scan<float, float, false>(p, n_requests, stream)
                        : launch_scan<bf16_t, bf16_t, false>(p, n_requests, stream);
}

// delta: q, k (rows of Hk*D, ld elements apart) and v (rows of H*Dv, ldv apart) of type dt (they
// may be parts of one wider row), after convolution and activation, not yet unit vectors; a float32
// [T][H*D] (overwritten with the decays); dt_bias float32 [H*D]; A_log float32 [H]; b float32, a token's H values
// ld_small apart; work arrays qn, kn float32 [T][H*D] and beta float32 [T][H]; state float32 [slots][H][D][Dv]; out
// float32 [T][H][Dv].  a_head (or null): one decay per head, its inputs a token's H values ld_small apart, dt_bias
// then [H]; a is then only written.
TUFF_EXPORT int tuff_delta_scan(const void* q, const void* k, const void* v, int dt, float* a, const float* dt_bias,
                                const float* A_log, const float* b, const float* a_head, long long ld_small, float* qn, float* kn,
                                float* beta, float* state, float* out, const int* q_start, const int* q_len, const int* state_slot,
                                int n_tokens, int n_requests, int H, int Hk, int D, int Dv, long long ld, long long ldv,
                                hipStream_t stream) {
    if (n_requests <= 0 || n_tokens <= 0) return 0;
    if (Hk <= 0 || H % Hk || H > 65535 || ld_small < H) return -2;
    PrepArgs pp{q, k, a, dt_bias, A_log, b, a_head, ld_small, qn, kn, beta, H, Hk, D, ld};
    if (dt == DT_F32) hipLaunchKernelGGL((scan_prep_kernel<float, true>), dim3(n_tokens, H), dim3(WAVE), 0, stream, pp);
    else hipLaunchKernelGGL((scan_prep_kernel<bf16_t, true>), dim3(n_tokens, H), dim3(WAVE), 0, stream, pp);
    ScanArgs p{qn, kn, v, a, beta, state, out, q_start, q_len, state_slot, H, H, D, Dv, ldv, (long long)H * D, nullptr};
    return dt == DT_F32 ? launch_scan<float, float, true>(p, n_requests, stream)
                        : launch_scan<float, bf16_t, true>(p, n_requests, stream);
}

// gate_dt: type of the gate's rows (float32 sums of a product may come in as they are), gate_ld elements apart; dt:
// type of y.  gate_first: the gate is applied before the norm.
TUFF_EXPORT int tuff_head_norm_gate(const float* o, const float* w, int w_stride, const void* gate, long long gate_ld, int gate_dt,
                                    int dt, int gate_fn, int gate_first, void* y, int n_tokens, int H, int Dv, float eps,
                                    hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (H > 65535 || (gate && gate_ld < (long long)H * Dv)) return -2;
    dim3 grid(n_tokens, H), block(WAVE);
    if (dt == DT_F32 && gate_dt == DT_F32) hipLaunchKernelGGL((head_norm_gate_kernel<float, float>), grid, block, 0, stream, o, w, w_stride, (const float*)gate, gate_ld, gate_fn, gate_first, (float*)y, H, Dv, eps);
    else if (gate_dt == DT_F32) hipLaunchKernelGGL((head_norm_gate_kernel<float, bf16_t>), grid, block, 0, stream, o, w, w_stride, (const float*)gate, gate_ld, gate_fn, gate_first, (bf16_t*)y, H, Dv, eps);
    else if (dt == DT_BF16) hipLaunchKernelGGL((head_norm_gate_kernel<bf16_t, bf16_t>), grid, block, 0, stream, o, w, w_stride, (const bf16_t*)gate, gate_ld, gate_fn, gate_first, (bf16_t*)y, H, Dv, eps);
    else return -2;
    return launch_status();
}

// ssd (the state-space recurrence with a scalar decay per head): xbc holds a token's convolved rows
// [x (H*P) | B (G*N) | C (G*N)] of type dt, ld elements apart; dt_raw float32, a token's H values ld_dt apart; dt_bias,
// A_log, Dh float32 [H]; work arrays step and decay float32 [T][H]; state float32 [slots][H][N][P]; out float32
// [T][H][P].  Head h reads B and C of group h / (H / G), from the rows as they lie.
TUFF_EXPORT int tuff_ssd_scan(const void* xbc, int dt, long long ld, const float* dt_raw, long long ld_dt, const float* dt_bias,
                              const float* A_log, const float* Dh, float* step, float* decay, float* state,
                              float* out, const int* q_start, const int* q_len, const int* state_slot, int n_tokens, int n_requests,
                              int H, int G, int N, int P, hipStream_t stream) {
    if (n_requests <= 0 || n_tokens <= 0) return 0;
    if (H <= 0 || H > 65535 || G <= 0 || H % G || ld < (long long)H * P + 2LL * G * N || ld_dt < H) return -2;
    const long long n = (long long)n_tokens * H;
    hipLaunchKernelGGL(ssd_prep_kernel, dim3((unsigned)ceil_div_ll(n, 256)), dim3(256), 0, stream, dt_raw, ld_dt, dt_bias, A_log, step, decay, (float*)nullptr, n, H);
    int rc = launch_status();
    if (rc != 0) return rc;
    const long long b_off = (long long)H * P, c_off = b_off + (long long)G * N;
    if (dt == DT_F32) {
        const float* x = (const float*)xbc;
        ScanArgs p{x + c_off, x + b_off, x, decay, step, state, out, q_start, q_len, state_slot, H, G, N, P, ld, ld, Dh};
        return launch_scan<float, float, false, false, true>(p, n_requests, stream);
    }
    const bf16_t* x = (const bf16_t*)xbc;
    ScanArgs p{x + c_off, x + b_off, x, decay, step, state, out, q_start, q_len, state_slot, H, G, N, P, ld, ld, Dh};
    return launch_scan<bf16_t, bf16_t, false, false, true>(p, n_requests, stream);
}

// The same recurrence in chunks of 64 tokens on the matrix cores (see above), for bfloat16 rows: N and P multiples of 16,
// N <= 128, P <= 64.  Work arrays: step, decay, log_decay float32 [T][H]; U float32 [chunks][H][N][P] and cdec float32
// [chunks][H] with chunks >= ceil(T / 64) + requests (what the step's portions can be cut into at most).
TUFF_EXPORT int tuff_ssd_chunked(const void* xbc, long long ld, const float* dt_raw, long long ld_dt, const float* dt_bias,
                                 const float* A_log, const float* Dh, float* step, float* decay, float* log_decay, float* U, float* cdec,
                                 int chunks, float* state, float* out, const int* q_start, const int* q_len, const int* state_slot,
                                 int n_tokens, int n_requests, int H, int G, int N, int P, hipStream_t stream) {
    if (n_requests <= 0 || n_tokens <= 0) return 0;
    if (H <= 0 || H > 65535 || G <= 0 || H % G || ld < (long long)H * P + 2LL * G * N || ld_dt < H) return -2;
    if (N % 16 || P % 16 || N > 128 || P > 64 || N <= 0 || P <= 0 || chunks < ceil_div(n_tokens, CHUNK) + n_requests || n_requests > 65535) return -2;
    const long long n = (long long)n_tokens * H;
    hipLaunchKernelGGL(ssd_prep_kernel, dim3((unsigned)ceil_div_ll(n, 256)), dim3(256), 0, stream, dt_raw, ld_dt, dt_bias, A_log, step, decay, log_decay, n, H);
    int rc = launch_status();
    if (rc != 0) return rc;
    SsdChunkArgs p{(const bf16_t*)xbc, ld, step, log_decay, Dh, state, U, cdec, out, q_start, q_len, state_slot, n_requests, H, G, N, P};
    if (ld % 8 || ((unsigned long long)xbc & 15)) return -2;         // the rows are read 16 bytes at a time
    const size_t lds1 = (size_t)(2 * CHUNK + (N + P) * (CHUNK + 4)) * sizeof(float);
    const size_t lds3 = (size_t)(2 * CHUNK + CHUNK * (CHUNK + 4)) * sizeof(float) + (size_t)(2 * CHUNK * (N + 8) + P * (CHUNK + 8)) * sizeof(bf16_t);
    if (lds1 > 65536 || lds3 > 65536) return -2;
    hipLaunchKernelGGL(ssd_chunk_state_kernel, dim3(chunks, H), dim3(256), lds1, stream, p);
    hipLaunchKernelGGL(ssd_state_pass_kernel, dim3(n_requests, H, (unsigned)ceil_div_ll((long long)N * P, 256)), dim3(256), 0, stream, p);
    hipLaunchKernelGGL(ssd_chunk_out_kernel, dim3(chunks, H), dim3(256), lds3, stream, p);
    return launch_status();
}

// forget: x rows [q (H*D) | z (H*D) | v (H*Dv)] of type dt, ld elements apart, as projected; bias (or null) and lower
// float32 [H*D]; work arrays qn, f float32 [T][H*D]; state float32 [slots][H][D][Dv]; out float32 [T][H][Dv].
TUFF_EXPORT int tuff_forget_scan(const void* x, int dt, long long ld, const float* bias, const float* lower, float* qn, float* f,
                                 float* state, float* out, const int* q_start, const int* q_len, const int* state_slot,
                                 int n_tokens, int n_requests, int H, int D, int Dv, hipStream_t stream) {
    if (n_requests <= 0 || n_tokens <= 0) return 0;
    if (H <= 0 || H > 65535 || ld < 2LL * H * D + (long long)H * Dv) return -2;
    const int HD = H * D;
    dim3 grid(n_tokens, ceil_div(HD, 256)), block(256);
    if (dt == DT_F32) hipLaunchKernelGGL(forget_prep_kernel<float>, grid, block, 0, stream, (const float*)x, ld, bias, lower, qn, f, HD);
    else hipLaunchKernelGGL(forget_prep_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)x, ld, bias, lower, qn, f, HD);
    int rc = launch_status();
    if (rc != 0) return rc;
    // (k and the per-token scalar are loaded and not used: they point at arrays of the right reach)
    const void* v = dt == DT_F32 ? (const void*)((const float*)x + 2LL * HD) : (const void*)((const bf16_t*)x + 2LL * HD);
    ScanArgs p{qn, qn, v, f, f, state, out, q_start, q_len, state_slot, H, H, D, Dv, ld, (long long)H * D, nullptr};
    return dt == DT_F32 ? launch_scan<float, float, false, true>(p, n_requests, stream)
                        : launch_scan<float, bf16_t, false, true>(p, n_requests, stream);
}
