// Linear recurrences with a diagonal decay: a per-head matrix state S [dk, dv] in fp32 that every token updates,
//   S <- diag(w) S + (c k) v^T,   o = S^T q  (+ d v),
// with a decay w per key channel (or one per head), a write strength c per head and token, and a skip weight d per head.
// Gated linear attention (w = a learned decay, c = 1), HGRN2 (w = f, k = 1 - f) and the state-space-duality layer of
// Mamba-2 (w = exp(-exp(A_log) dt) per head, c = dt, k = B, q = C, v = x, d = D; B and C shared by the heads of a group)
// are all this one scan; what differs is how the operands are made from the projections:
//   nvh_hgrn2_prep / nvh_gla_prep / nvh_ssd_conv_prep   projection rows (type A) -> fp32 operands; the last also runs the
//                    short causal convolution over [x | B | C] with the sequence's carried inputs, silu, softplus of dt
//   nvh_conv_state_update   leaves the last taps-1 convolution inputs of every sequence in its state slot
//   nvh_gated_linear_scan   the recurrence: state columns spread over (sequence, head, column block), each column held by
//                    16 lanes (4 when dk is no multiple of 16) in registers, operands staged through LDS a stage ahead.
//                    The order of every sum is fixed by the sizes alone: one piece, portions or single tokens give the
//                    same bits.
//   nvh_group_rmsnorm_gate  read-out: RMS norm over groups of columns, weight, and a silu / sigmoid gate before or after.
// Everything that enters the recurrence is fp32; A (bf16 or fp32) is the type of projections, weights and results.
#include <algorithm>
#include "common.h"

namespace {

template <typename A>
__device__ __forceinline__ float ldf(const A* p, int64_t i) {
    return (float)p[i];
}
__device__ __forceinline__ float sigmoid_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float silu_(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float logsigmoid_(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// The sequence that owns packed token t (cu: [batch + 1] ascending; null: token t is sequence t).
__device__ __forceinline__ int seq_of_token(const int32_t* cu, int batch, int64_t t) {
    if (!cu) return (int)t;
    int lo = 0, hi = batch - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (cu[mid] <= t) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

// ---------------------------------------------------------------------------------------------------------------
struct Hgrn2PrepArgs {
    const void *q, *f, *v;     // projection columns [T, H dk], [T, H dk], [T, H dv]
    int64_t q_stride, f_stride, v_stride;
    const void *f_bias, *lower;     // [H dk]
    float *oq, *ok, *ow, *ov;  // fp32 [T, H dk] x 3, [T, H dv]
    int64_t n_k, n_v;
};

template <typename A>
__global__ __launch_bounds__(256) void hgrn2_prep_kernel(Hgrn2PrepArgs p) {
    const int64_t t = blockIdx.x;
    for (int64_t i = threadIdx.x; i < p.n_k; i += 256) {
        const float lo = ldf((const A*)p.lower, i);
        const float f = lo + (1.0f - lo) * sigmoid_(ldf((const A*)p.f, t * p.f_stride + i) + ldf((const A*)p.f_bias, i));
        p.oq[t * p.n_k + i] = silu_(ldf((const A*)p.q, t * p.q_stride + i));
        p.ow[t * p.n_k + i] = f;
        p.ok[t * p.n_k + i] = 1.0f - f;
    }
    for (int64_t i = threadIdx.x; i < p.n_v; i += 256) p.ov[t * p.n_v + i] = ldf((const A*)p.v, t * p.v_stride + i);
}

struct GlaPrepArgs {
    const void *q, *k, *v;     // projection columns
    int64_t q_stride, k_stride, v_stride;
    const float* z;            // fp32 decay logits [T, H dk]
    int64_t z_stride;
    float q_scale, inv_tau;
    float *oq, *ok, *ow, *ov;
    int64_t n_k, n_v;
};

template <typename A>
__global__ __launch_bounds__(256) void gla_prep_kernel(GlaPrepArgs p) {
    const int64_t t = blockIdx.x;
    for (int64_t i = threadIdx.x; i < p.n_k; i += 256) {
        p.oq[t * p.n_k + i] = ldf((const A*)p.q, t * p.q_stride + i) * p.q_scale;
        p.ok[t * p.n_k + i] = ldf((const A*)p.k, t * p.k_stride + i);
        p.ow[t * p.n_k + i] = expf(logsigmoid_(p.z[t * p.z_stride + i]) * p.inv_tau);      // sigmoid(z)^(1/tau)
    }
    for (int64_t i = threadIdx.x; i < p.n_v; i += 256) p.ov[t * p.n_v + i] = ldf((const A*)p.v, t * p.v_stride + i);
}

// The operands of the RWKV time mix from its projections: r, k, v as they are and the decay of every key channel,
//   w = exp(-exp(w0 + W2 tanh(l))),   l: the token's low-rank decay input [rank], W2 [n_k, rank],
// with the rank-sized product inside (fp32 throughout; tanh(l) sits in LDS).
struct WkvPrepArgs {
    const void *r, *k, *v, *l;
    int64_t r_stride, k_stride, v_stride, l_stride;
    const void *w2, *w0;
    float *oq, *ok, *ow, *ov;
    int64_t n_k, n_v;
    int rank;
};

template <typename A>
__global__ __launch_bounds__(256) void wkv_prep_kernel(WkvPrepArgs p) {
    extern __shared__ float th[];
    const int64_t t = blockIdx.x;
    for (int j = threadIdx.x; j < p.rank; j += 256) th[j] = tanhf(ldf((const A*)p.l, t * p.l_stride + j));
    __syncthreads();
    for (int64_t i = threadIdx.x; i < p.n_k; i += 256) {
        const A* wr = (const A*)p.w2 + i * p.rank;
        float z = ldf((const A*)p.w0, i);
        for (int j = 0; j < p.rank; ++j) z = __builtin_fmaf((float)wr[j], th[j], z);
        p.oq[t * p.n_k + i] = ldf((const A*)p.r, t * p.r_stride + i);
        p.ok[t * p.n_k + i] = ldf((const A*)p.k, t * p.k_stride + i);
        p.ow[t * p.n_k + i] = expf(-expf(z));
    }
    for (int64_t i = threadIdx.x; i < p.n_v; i += 256) p.ov[t * p.n_v + i] = ldf((const A*)p.v, t * p.v_stride + i);
}

// ---------------------------------------------------------------------------------------------------------------
// Token shift: every token's input h is blended with the input of the token before it, with a weight vector per consumer,
//   out[s, t, :] = h_t + (h_(t-1) - h_t) mu[s, :],   s = 0 .. n - 1,
// where h_(t-1) of a step's first token is the input the sequence's slot carries (zeros at a sequence's start).  The
// slot is brought up to date by nvh_conv_state_update afterwards (the carried input of a convolution with two taps).
struct ShiftArgs {
    const void* h;             // [T, D]
    int64_t h_stride;
    const float* state;        // [slots, D]
    const int32_t *slots, *cu_seqlens_q, *context_lens;
    int batch;
    const void* mu;            // [n, D]
    void* out;                 // [n, T, D]
    int64_t tokens;
    int n, D, vec;
};

template <typename A>
__global__ __launch_bounds__(256) void token_shift_mix_kernel(ShiftArgs p) {
    const int64_t t = blockIdx.x;
    const int seq = seq_of_token(p.cu_seqlens_q, p.batch, t);
    const int lo = p.cu_seqlens_q ? p.cu_seqlens_q[seq] : seq, hi = p.cu_seqlens_q ? p.cu_seqlens_q[seq + 1] : seq + 1;
    const int slot = p.slots[seq];
    const bool first = (int)t == lo;
    const bool carried = slot >= 0 && p.context_lens[seq] != hi - lo;
    const A* cur = (const A*)p.h + t * p.h_stride;
    const A* prev = first ? nullptr : cur - p.h_stride;
    const float* st = first && carried ? p.state + (int64_t)slot * p.D : nullptr;
    if (p.vec) {                                             // eight consecutive columns per lane, 16-byte accesses
        for (int i = threadIdx.x * 8; i < p.D; i += 256 * 8) {
            float c[8], b[8];
            nvh_load8(cur, i, 8, true, c);
            if (prev) {
                nvh_load8(prev, i, 8, true, b);
            } else if (st) {
                nvh_load8(st, i, 8, true, b);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) b[e] = 0.f;
            }
            for (int s = 0; s < p.n; ++s) {
                float m[8];
                nvh_load8((const A*)p.mu, (int64_t)s * p.D + i, 8, true, m);
                A* dst = (A*)p.out + ((int64_t)s * p.tokens + t) * p.D + i;
                if constexpr (sizeof(A) == 2) {
                    bf16x8 o;
#pragma unroll
                    for (int e = 0; e < 8; ++e) o[e] = (bf16)(c[e] + (b[e] - c[e]) * m[e]);
                    *reinterpret_cast<bf16x8*>(dst) = o;
                } else {
                    f32x4 lo4, hi4;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        lo4[e] = c[e] + (b[e] - c[e]) * m[e];
                        hi4[e] = c[4 + e] + (b[4 + e] - c[4 + e]) * m[4 + e];
                    }
                    *reinterpret_cast<f32x4*>(dst) = lo4;
                    *reinterpret_cast<f32x4*>(dst + 4) = hi4;
                }
            }
        }
        return;
    }
    for (int i = threadIdx.x; i < p.D; i += 256) {
        const float c = (float)cur[i];
        const float b = prev ? (float)prev[i] : (st ? st[i] : 0.f);
        const float d = b - c;
        for (int s = 0; s < p.n; ++s)
            ((A*)p.out)[((int64_t)s * p.tokens + t) * p.D + i] = (A)(c + d * (float)((const A*)p.mu)[(int64_t)s * p.D + i]);
    }
}

// q, k, v projection columns -> the scan's fp32 operands with rotary positions on the first rot_dims dimensions of every q
// and k head (angle = position * freq[pair], cos and sin times `mag`), q and k scaled AFTER the rotation.
struct RotPrepArgs {
    const void *q, *k, *v;
    int64_t q_stride, k_stride, v_stride;
    const int64_t* positions;
    const float* freq;         // [rot_dims / 2] or null (rot_dims 0)
    float mag, q_scale, k_scale;
    int rot_dims, interleaved, H, dim, vdim;
    float *oq, *ok, *ov;
};

template <typename A>
__global__ __launch_bounds__(256) void rotary_qkv_prep_kernel(RotPrepArgs a) {
    const int64_t t = blockIdx.x;
    const float pos = (float)a.positions[t];
    const int nk = a.H * a.dim, nv = a.H * a.vdim;
    for (int which = 0; which < 2; ++which) {
        const A* src = (const A*)(which ? a.k : a.q) + t * (which ? a.k_stride : a.q_stride);
        float* dst = (which ? a.ok : a.oq) + t * nk;
        const float scale = which ? a.k_scale : a.q_scale;
        for (int i = threadIdx.x; i < nk; i += 256) {
            const int d = i % a.dim;
            float v = (float)src[i];
            if (d < a.rot_dims) {
                int partner, pair;
                bool first;
                pair_of(d, a.rot_dims, a.interleaved, partner, pair, first);
                const float o = (float)src[i - d + partner];
                float sn, cs;
                rot_sincos<A>(pos * a.freq[pair], sn, cs);
                const float c = cs * a.mag, s = sn * a.mag;
                v = first ? v * c - o * s : v * c + o * s;
            }
            dst[i] = v * scale;
        }
    }
    const A* vr = (const A*)a.v + t * a.v_stride;
    for (int i = threadIdx.x; i < nv; i += 256) a.ov[t * nv + i] = (float)vr[i];
}

// ---------------------------------------------------------------------------------------------------------------
struct SsdPrepArgs {
    const void* xbc;           // [T, ld]: the convolved channels of the in-projection row: x (H dv wide), then B and C (G N wide each)
    int64_t xbc_stride;
    const void* dt;            // [T, ld]: H columns
    int64_t dt_stride;
    const void *conv_w, *conv_b;    // [C, taps], [C] (null: no bias)
    const void *dt_bias, *a_log;    // [H]
    float* conv_state;         // [slots, taps - 1, C]: the inputs of the sequence's last taps - 1 tokens, oldest first
    const int32_t *slots, *cu_seqlens_q, *context_lens;
    int batch, taps, H, inner, gn;  // inner = H dv, gn = G N; C = inner + 2 gn
    float *ov, *ok, *oq, *oc, *ow;  // fp32 [T, inner], [T, gn] (B), [T, gn] (C), [T, H] (dt), [T, H] (decay)
};

template <typename A>
__global__ __launch_bounds__(256) void ssd_conv_prep_kernel(SsdPrepArgs p) {
    const int64_t t = blockIdx.x;
    const int seq = seq_of_token(p.cu_seqlens_q, p.batch, t);
    const int lo = p.cu_seqlens_q ? p.cu_seqlens_q[seq] : seq, hi = p.cu_seqlens_q ? p.cu_seqlens_q[seq + 1] : seq + 1;
    const int j = (int)t - lo;                               // index of the token among this step's tokens of its sequence
    const int slot = p.slots[seq];
    const bool carried = slot >= 0 && p.context_lens[seq] != hi - lo;       // inputs from before this step exist
    const int C = p.inner + 2 * p.gn, taps = p.taps;
    const float* st = carried ? p.conv_state + (int64_t)slot * (taps - 1) * C : nullptr;
    for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += 256 * gridDim.y) {
        float acc = p.conv_b ? ldf((const A*)p.conv_b, c) : 0.f;
        for (int k = 0; k < taps; ++k) {                     // tap k multiplies the input taps - 1 - k tokens back
            const int back = taps - 1 - k, src = j - back;
            float in = 0.f;
            if (src >= 0) in = ldf((const A*)p.xbc, (t - back) * p.xbc_stride + c);
            else if (st) in = st[(int64_t)(taps - 1 + src) * C + c];
            acc = __builtin_fmaf(ldf((const A*)p.conv_w, (int64_t)c * taps + k), in, acc);
        }
        const float y = silu_(acc);
        if (c < p.inner) p.ov[t * p.inner + c] = y;
        else if (c < p.inner + p.gn) p.ok[t * p.gn + (c - p.inner)] = y;
        else p.oq[t * p.gn + (c - p.inner - p.gn)] = y;
    }
    if (blockIdx.y != 0) return;
    for (int h = threadIdx.x; h < p.H; h += 256) {
        const float dt = softplus_(ldf((const A*)p.dt, t * p.dt_stride + h) + ldf((const A*)p.dt_bias, h));
        p.oc[t * p.H + h] = dt;
        p.ow[t * p.H + h] = expf(-expf(ldf((const A*)p.a_log, h)) * dt);
    }
}

// The same with eight consecutive channels per lane and 16-byte accesses (TAPS known at compile time; channel counts of x, B, C
// multiples of 8, rows 16-byte aligned): a tap is one load of the inputs and one of the weights instead of eight of each.
template <typename A, int TAPS>
__global__ __launch_bounds__(256) void ssd_conv_prep_vec_kernel(SsdPrepArgs p) {
    const int64_t t = blockIdx.x;
    const int seq = seq_of_token(p.cu_seqlens_q, p.batch, t);
    const int lo = p.cu_seqlens_q ? p.cu_seqlens_q[seq] : seq, hi = p.cu_seqlens_q ? p.cu_seqlens_q[seq + 1] : seq + 1;
    const int j = (int)t - lo;
    const int slot = p.slots[seq];
    const bool carried = slot >= 0 && p.context_lens[seq] != hi - lo;
    const int C = p.inner + 2 * p.gn;
    const float* st = carried ? p.conv_state + (int64_t)slot * (TAPS - 1) * C : nullptr;
    for (int c = (blockIdx.y * 256 + threadIdx.x) * 8; c < C; c += 256 * 8 * gridDim.y) {
        float acc[8], wf[8 * TAPS];                          // wf[i * TAPS + k]: channel c + i, tap k (as the weights lie)
        if (p.conv_b) {
            nvh_load8((const A*)p.conv_b, c, 8, true, acc);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = 0.f;
        }
#pragma unroll
        for (int k = 0; k < TAPS; ++k) {
            float piece[8];
            nvh_load8((const A*)p.conv_w, (int64_t)c * TAPS + 8 * k, 8, true, piece);
#pragma unroll
            for (int i = 0; i < 8; ++i) wf[8 * k + i] = piece[i];
        }
#pragma unroll
        for (int k = 0; k < TAPS; ++k) {                     // tap k multiplies the input TAPS - 1 - k tokens back
            const int back = TAPS - 1 - k, src = j - back;
            float in[8];
            if (src >= 0) {
                nvh_load8((const A*)p.xbc, (t - back) * p.xbc_stride + c, 8, true, in);
            } else if (st) {
                nvh_load8(st, (int64_t)(TAPS - 1 + src) * C + c, 8, true, in);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) in[i] = 0.f;
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(wf[i * TAPS + k], in[i], acc[i]);
        }
        float* dst = c < p.inner ? p.ov + t * p.inner + c : (c < p.inner + p.gn ? p.ok + t * p.gn + (c - p.inner) : p.oq + t * p.gn + (c - p.inner - p.gn));
        f32x4 lo4, hi4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            lo4[i] = silu_(acc[i]);
            hi4[i] = silu_(acc[4 + i]);
        }
        *reinterpret_cast<f32x4*>(dst) = lo4;
        *reinterpret_cast<f32x4*>(dst + 4) = hi4;
    }
    if (blockIdx.y != 0) return;
    for (int h = threadIdx.x; h < p.H; h += 256) {
        const float dt = softplus_(ldf((const A*)p.dt, t * p.dt_stride + h) + ldf((const A*)p.dt_bias, h));
        p.oc[t * p.H + h] = dt;
        p.ow[t * p.H + h] = expf(-expf(ldf((const A*)p.a_log, h)) * dt);
    }
}

// One thread per (sequence, channel): slot s of the new state is input number n + s - (taps - 1) of [carried | this step's].
// Ascending s only ever reads carried entries at or above the one it writes.
template <typename A>
__global__ __launch_bounds__(256) void conv_state_update_kernel(SsdPrepArgs p) {
    const int seq = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    const int C = p.inner + 2 * p.gn, keep = p.taps - 1;
    const int slot = p.slots[seq];
    if (slot < 0 || c >= C) return;
    const int lo = p.cu_seqlens_q ? p.cu_seqlens_q[seq] : seq, hi = p.cu_seqlens_q ? p.cu_seqlens_q[seq + 1] : seq + 1;
    const int n = hi - lo;
    if (n <= 0) return;
    const bool carried = p.context_lens[seq] != n;
    float* st = p.conv_state + (int64_t)slot * keep * C;
    for (int s = 0; s < keep; ++s) {
        const int src = n + s - keep;
        float v = 0.f;
        if (src >= 0) v = ldf((const A*)p.xbc, (int64_t)(lo + src) * p.xbc_stride + c);
        else if (carried) v = st[(int64_t)(s + n) * C + c];
        st[(int64_t)s * C + c] = v;
    }
}

// The residual stream plus its own short causal convolution over time, per column: h_t = x_t + sum_k w[:, k] x_(t - taps + 1 + k), the
// last tap on the token itself, zeros before the sequence's start, continued across steps from the sequence's carried rows
// (state [slots, taps - 1, dim], brought up to date by nvh_conv_state_update afterwards).  x and the sums are fp32; h leaves in
// the activation type.  One workgroup per token.
struct StreamConvArgs {
    const float* x;            // [T, dim]
    const void* w;             // [dim, taps]
    const float* state;
    const int32_t *slots, *cu_seqlens_q, *context_lens;
    void* h;
    int64_t h_stride;
    int batch, taps, dim;
};

template <typename A>
__global__ __launch_bounds__(256) void stream_conv_kernel(StreamConvArgs p) {
    const int64_t t = blockIdx.x;
    const int seq = seq_of_token(p.cu_seqlens_q, p.batch, t);
    const int lo = p.cu_seqlens_q ? p.cu_seqlens_q[seq] : seq, hi = p.cu_seqlens_q ? p.cu_seqlens_q[seq + 1] : seq + 1;
    const int j = (int)t - lo, taps = p.taps, dim = p.dim;
    const int slot = p.slots[seq];
    const bool carried = slot >= 0 && p.context_lens[seq] != hi - lo;
    const float* st = carried ? p.state + (int64_t)slot * (taps - 1) * dim : nullptr;
    A* h = (A*)p.h + t * p.h_stride;
    for (int c = blockIdx.y * 256 + threadIdx.x; c < dim; c += 256 * gridDim.y) {
        const float cur = p.x[t * dim + c];
        float acc = 0.f;
        for (int k = 0; k < taps; ++k) {
            const int back = taps - 1 - k, src = j - back;
            float in = 0.f;
            if (src >= 0) in = p.x[(t - back) * dim + c];
            else if (st) in = st[(int64_t)(taps - 1 + src) * dim + c];
            acc = __builtin_fmaf(ldf((const A*)p.w, (int64_t)c * taps + k), in, acc);
        }
        h[c] = (A)(cur + acc);
    }
}

// ---------------------------------------------------------------------------------------------------------------
struct ScanArgs {
    const float *q, *k;        // [T, QG, dk]: head h reads group h / (H / QG)
    int64_t q_stride, k_stride;
    int qk_groups;
    const float* w;            // decay: [T, H, dk], or [T, H] when w_scalar
    int64_t w_stride;
    int w_scalar;
    const float* kscale;       // [T, H] or null (1)
    int64_t ks_stride;
    const float* v;            // [T, H, dv]
    int64_t v_stride;
    const float* skip;         // [H] or null
    float* state;              // [slots, H, dv, dk] (the memory S transposed: a column's dk rows are contiguous)
    const int32_t *slots, *cu_seqlens_q, *context_lens;
    float* out;                // [T, H dv]
    int H, dk, dv;
    int nseg, seg_min;         // segments per long portion (1: none) and the fewest tokens that are cut
    float *ws_l, *ws_d;        // records of the segments: end states [batch, H, nseg, dv, dk] and decay products [batch, H, nseg, dk]
    const float* bonus;        // PRE only: [H, dk] or null (0)
};

// Lanes per state column (SUBS), rows held per lane (DKQ), EXACT: dk == DKQ * SUBS (no loop carries a run-time bound; rows
// beyond dk are held as zeros otherwise).  A workgroup owns
// COLS = 256 / SUBS columns of one (sequence, head).  A token's staged row: q (dk) | k (dk) | w (dk) | v (COLS) | c | padding.
//
// MODE 0: a sequence's tokens of this step are walked in one go.
// MODE 1 and 2, for long portions (a token costs the chain S -> S whatever the chip has idle): the portion is cut into
// `nseg` segments that are walked side by side.  MODE 1 walks every segment from a zero state (the first from the
// sequence's state), writes the outputs that this gives, and leaves per segment its end state L_j and the product D_j of
// its decays.  MODE 2 gives segment j >= 1 what it missed: its true start S_j = D_(j-1) S_(j-1) + L_(j-1), S_1 = L_0,
// folded from the records, adds (P_t q_t)^T S_j to every output of the segment (P_t: the product of the segment's decays
// up to t), and the last segment leaves the sequence's state.  Products only, no division: a decay that underflows is a
// zero.  A sequence with fewer than `seg_min` tokens in the step is one segment (MODE 1 then does all of it).
//
// PRE: the token is read out BEFORE it is written and decayed, with a bonus u per key channel for the token itself,
//   o = (S + diag(u) (c k) v^T)^T q (+ d v),   S <- diag(w) S + (c k) v^T,
// the form of the RWKV time mix.  The joining launch then weighs a segment's start state by the decays BEFORE the token.
template <int DKQ, int SUBS, bool EXACT, int MODE, bool PRE>
__global__ __launch_bounds__(256) void gated_linear_scan_kernel(ScanArgs p) {
    constexpr int COLS = 256 / SUBS;
    constexpr int CH = (3 * DKQ * SUBS + COLS + 4 + 255) / 256;     // loads per lane and token
    constexpr int TOK = (32 / CH) < 2 ? 2 : (32 / CH);
    extern __shared__ __attribute__((aligned(16))) float sm[];
    const int seq = blockIdx.x, head = blockIdx.y;
    const int dk = p.dk, dv = p.dv, dkq = (dk + SUBS - 1) / SUBS;
    const int seg = MODE == 0 ? 0 : (int)blockIdx.z % p.nseg, colblock = MODE == 0 ? (int)blockIdx.z : (int)blockIdx.z / p.nseg;
    const int col0 = colblock * COLS, lcol = threadIdx.x / SUBS, col = col0 + lcol, sub = threadIdx.x % SUBS;
    const bool live = col < dv;
    const int seq_lo = p.cu_seqlens_q ? p.cu_seqlens_q[seq] : seq, seq_hi = p.cu_seqlens_q ? p.cu_seqlens_q[seq + 1] : seq + 1;
    const int slot = p.slots[seq];
    if (slot < 0 || seq_hi <= seq_lo) return;                // a padded row (uniform over the workgroup)
    const int nseg = (MODE != 0 && seq_hi - seq_lo >= p.seg_min) ? p.nseg : 1;
    if (seg >= nseg || (MODE == 2 && seg == 0)) return;      // (uniform)
    const int seg_len = (seq_hi - seq_lo + nseg - 1) / nseg;
    const int lo = seq_lo + seg * seg_len, hi = min(seq_hi, lo + seg_len);   // (hi <= lo: an empty segment; it still leaves its records)
    const bool fresh = p.context_lens[seq] == seq_hi - seq_lo;
    float* sp = p.state + (((int64_t)slot * p.H + head) * dv) * dk;      // [dv, dk]: a column's rows lie together
    const int64_t rec = ((int64_t)seq * p.H + head) * p.nseg;            // this (sequence, head)'s first record
    // Rows of a lane: with 16-byte LDS reads (EXACT, DKQ a multiple of 4) lane `sub` takes rows 4 sub .. 4 sub + 3 of every 64, so the
    // 16 lanes of a column read 256 consecutive bytes at a time; otherwise every SUBS-th row, consecutive floats across the lanes.
    constexpr bool VEC4 = EXACT && DKQ % 4 == 0;
    auto row_of = [&](int ii) { return VEC4 ? 4 * SUBS * (ii >> 2) + 4 * sub + (ii & 3) : SUBS * ii + sub; };
    auto row_ok = [&](int ii) { return EXACT || row_of(ii) < dk; };
    float S[DKQ], P[DKQ], U[PRE ? DKQ : 1];
    if constexpr (PRE) {
#pragma unroll
        for (int ii = 0; ii < DKQ; ++ii) U[ii] = (p.bonus && row_ok(ii)) ? p.bonus[(int64_t)head * dk + row_of(ii)] : 0.f;
    }
#pragma unroll
    for (int ii = 0; ii < DKQ; ++ii) {
        P[ii] = 1.f;
        S[ii] = 0.f;
        if (MODE != 2 && seg == 0 && live && !fresh && row_ok(ii)) S[ii] = sp[(int64_t)col * dk + row_of(ii)];
    }
    if constexpr (MODE == 2) {
        // the state this segment starts from, folded from the records of the segments before it
        for (int j = 0; j < seg; ++j) {
            const float* lj = p.ws_l + ((rec + j) * dv + col) * dk;
            const float* dj = p.ws_d + (rec + j) * dk;
#pragma unroll
            for (int ii = 0; ii < DKQ; ++ii)
                if (live && row_ok(ii)) S[ii] = __builtin_fmaf(dj[row_of(ii)], S[ii], lj[row_of(ii)]);
        }
    }
    const int rowf = (3 * dk + COLS + 4) & ~3;             // (a multiple of 4 floats: rows stay 16-byte aligned)
    float* osm = sm + TOK * rowf;                            // [TOK][COLS]: the stage's outputs
    const int group = head / (p.H / p.qk_groups);
    const float* qb = p.q + (int64_t)group * dk;
    const float* kb = p.k + (int64_t)group * dk;
    const float* wb = p.w + (p.w_scalar ? (int64_t)head : (int64_t)head * dk);
    const float* vb = p.v + (int64_t)head * dv;
    const float skip = p.skip ? p.skip[head] : 0.f;
    float pre[TOK][CH];
    auto fetch = [&](int t0) {
#pragma unroll
        for (int tt = 0; tt < TOK; ++tt) {
            const int64_t tok = t0 + tt;
            if (tok < hi)                                    // (uniform; a one-token step loads one row, not TOK copies of it)
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int e = min((int)threadIdx.x + 256 * c, rowf - 1);
                float x;
                if (e < dk) x = qb[tok * p.q_stride + e];
                else if (e < 2 * dk) x = kb[tok * p.k_stride + (e - dk)];
                else if (e < 3 * dk) x = wb[tok * p.w_stride + (p.w_scalar ? 0 : e - 2 * dk)];
                else if (e < 3 * dk + COLS) x = vb[tok * p.v_stride + min(col0 + e - 3 * dk, dv - 1)];
                else x = p.kscale ? p.kscale[tok * p.ks_stride + head] : 1.0f;
                pre[tt][c] = x;
            }
        }
    };
    if (lo < hi) fetch(lo);
    for (int t0 = lo; t0 < hi; t0 += TOK) {
        const int nt = min(TOK, hi - t0);
        __syncthreads();                                     // the previous stage's readers are done
#pragma unroll
        for (int tt = 0; tt < TOK; ++tt)
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int e = threadIdx.x + 256 * c;
                if (e < rowf) sm[tt * rowf + e] = pre[tt][c];
            }
        __syncthreads();
        if (t0 + TOK < hi) fetch(t0 + TOK);
        // A token's operands are read from LDS one token ahead, into the register set the other token is not using, so the
        // reads' latency is off the chain S -> S.
        auto read_token = [&](int tt, float (&xq)[DKQ], float (&xk)[DKQ], float (&xw)[DKQ], float& xv, float& xs) {
            const float* row = sm + tt * rowf;
            if constexpr (VEC4) {
#pragma unroll
                for (int c4 = 0; c4 < DKQ / 4; ++c4) {
                    const int i = 4 * SUBS * c4 + 4 * sub;
                    const f32x4 vq = *reinterpret_cast<const f32x4*>(row + i), vw = *reinterpret_cast<const f32x4*>(row + 2 * dk + i);
                    f32x4 vk = {0.f, 0.f, 0.f, 0.f};
                    if constexpr (MODE != 2) vk = *reinterpret_cast<const f32x4*>(row + dk + i);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        xq[4 * c4 + e] = vq[e];
                        xk[4 * c4 + e] = vk[e];
                        xw[4 * c4 + e] = vw[e];
                    }
                }
            } else {
#pragma unroll
                for (int ii = 0; ii < DKQ; ++ii)
                    if (EXACT || ii < dkq) {
                        const int i = row_of(ii);
                        const bool in = EXACT || i < dk;     // (a row beyond dk: its state stays zero)
                        xq[ii] = in ? row[i] : 0.f;
                        xk[ii] = in && MODE != 2 ? row[dk + i] : 0.f;
                        xw[ii] = in ? row[2 * dk + i] : 0.f;
                    }
            }
            xv = row[3 * dk + lcol];
            xs = row[3 * dk + COLS];
        };
        auto token = [&](int tt, const float (&xq)[DKQ], const float (&xk)[DKQ], const float (&xw)[DKQ], float xv, float xs) {
            const float sv = xs * xv;
            float o = 0.f;
#pragma unroll
            for (int ii = 0; ii < DKQ; ++ii)
                if (EXACT || ii < dkq) {
                    if constexpr (MODE == 2) {
                        if constexpr (PRE) {
                            o = __builtin_fmaf(P[ii] * xq[ii], S[ii], o);
                            P[ii] *= xw[ii];
                        } else {
                            P[ii] *= xw[ii];
                            o = __builtin_fmaf(P[ii] * xq[ii], S[ii], o);
                        }
                    } else if constexpr (PRE) {
                        const float kv = xk[ii] * sv;
                        o = __builtin_fmaf(__builtin_fmaf(U[ii], kv, S[ii]), xq[ii], o);
                        S[ii] = __builtin_fmaf(xw[ii], S[ii], kv);
                        if constexpr (MODE == 1) P[ii] *= xw[ii];
                    } else {
                        const float sn = __builtin_fmaf(xw[ii], S[ii], xk[ii] * sv);
                        S[ii] = sn;
                        o = __builtin_fmaf(sn, xq[ii], o);
                        if constexpr (MODE == 1) P[ii] *= xw[ii];
                    }
                }
            if constexpr (SUBS == 16) {
                o = row16_sum(o);
            } else {
                o += NVH_DPP(o, 0xB1);
                o += NVH_DPP(o, 0x4E);
            }
            if (sub == 0) osm[tt * COLS + lcol] = MODE == 2 ? o : __builtin_fmaf(skip, xv, o);
        };
        float cq[DKQ], ck[DKQ], cw[DKQ], cv, cs, nq[DKQ], nk[DKQ], nw[DKQ], nv, ns;
        read_token(0, cq, ck, cw, cv, cs);
        int tt = 0;
        for (; tt + 1 < nt; tt += 2) {
            read_token(tt + 1, nq, nk, nw, nv, ns);
            token(tt, cq, ck, cw, cv, cs);
            read_token(min(tt + 2, TOK - 1), cq, ck, cw, cv, cs);
            token(tt + 1, nq, nk, nw, nv, ns);
        }
        if (tt < nt) token(tt, cq, ck, cw, cv, cs);
        // the stage's outputs leave together, a token's columns side by side (MODE 2 adds to what MODE 1 wrote)
        __syncthreads();
        for (int i = threadIdx.x; i < nt * COLS; i += 256) {
            const int ot = i / COLS, oc = i - ot * COLS;
            if (col0 + oc < dv) {
                float* dst = p.out + (int64_t)(t0 + ot) * p.H * dv + head * dv + col0 + oc;
                if constexpr (MODE == 2) *dst += osm[i];
                else *dst = osm[i];
            }
        }
    }
    if constexpr (MODE == 2) {
        if (seg != nseg - 1) return;
        // the last segment: the sequence's state after this step, D S + L with its own record
        const float* lj = p.ws_l + ((rec + seg) * dv + col) * dk;
#pragma unroll
        for (int ii = 0; ii < DKQ; ++ii)
            if (live && row_ok(ii)) S[ii] = __builtin_fmaf(P[ii], S[ii], lj[row_of(ii)]);
    }
    if (MODE == 1 && nseg > 1) {
        if (live) {
            float* lj = p.ws_l + ((rec + seg) * dv + col) * dk;
#pragma unroll
            for (int ii = 0; ii < DKQ; ++ii)
                if (row_ok(ii)) lj[row_of(ii)] = S[ii];
        }
        if (colblock == 0 && lcol == 0) {
#pragma unroll
            for (int ii = 0; ii < DKQ; ++ii)
                if (row_ok(ii)) p.ws_d[(rec + seg) * dk + row_of(ii)] = P[ii];
        }
        return;
    }
    if (live) {
#pragma unroll
        for (int ii = 0; ii < DKQ; ++ii)
            if (row_ok(ii)) sp[(int64_t)col * dk + row_of(ii)] = S[ii];
    }
}

// ---------------------------------------------------------------------------------------------------------------
// y[t, g, :] = unit(o') w (* gate afterwards), o' = o (* gate beforehand); one wave per (token, group of `gs` columns).
// weight: [gs] shared by the groups (w_full 0) or [groups gs] (w_full 1).  gate_act: 0 none, 1 sigmoid, 2 silu.
template <typename A>
__global__ __launch_bounds__(256) void group_rmsnorm_gate_kernel(const float* __restrict__ o, const A* __restrict__ weight, int w_full, const A* __restrict__ gate,
                                                                 int64_t gate_stride, int gate_act, int gate_first, A* __restrict__ y, int64_t y_stride,
                                                                 int64_t rows, int groups, int gs, float eps) {
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= rows * groups) return;
    const int64_t t = item / groups;
    const int g = (int)(item - t * groups), lane = threadIdx.x & 63;
    const float* orow = o + (t * groups + g) * gs;
    auto gate_of = [&](int i) {
        const float z = ldf(gate, t * gate_stride + (int64_t)g * gs + i);
        return gate_act == 1 ? sigmoid_(z) : silu_(z);
    };
    const bool pre = gate && gate_act && gate_first, post = gate && gate_act && !gate_first;
    float ss = 0.f;
    for (int i = lane; i < gs; i += 64) {
        const float v = pre ? orow[i] * gate_of(i) : orow[i];
        ss += v * v;
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
    for (int i = lane; i < gs; i += 64) {
        float v = pre ? orow[i] * gate_of(i) : orow[i];
        v = v * inv * (weight ? ldf(weight, w_full ? (int64_t)g * gs + i : i) : 1.0f);
        if (post) v *= gate_of(i);
        y[t * y_stride + (int64_t)g * gs + i] = (A)v;
    }
}

// The same with one workgroup per (token, group), for groups of more than 256 columns (up to 256 PER): the gated values stay
// in registers between the sum and the write.
template <typename A, int PER>
__global__ __launch_bounds__(256) void group_rmsnorm_gate_block_kernel(const float* __restrict__ o, const A* __restrict__ weight, int w_full, const A* __restrict__ gate,
                                                                       int64_t gate_stride, int gate_act, int gate_first, A* __restrict__ y, int64_t y_stride,
                                                                       int groups, int gs, float eps) {
    __shared__ float red[4];
    const int64_t t = blockIdx.x / groups;
    const int g = (int)(blockIdx.x - t * groups);
    const float* orow = o + (t * groups + g) * gs;
    const A* grow = gate ? gate + t * gate_stride + (int64_t)g * gs : nullptr;
    const bool pre = gate && gate_act && gate_first, post = gate && gate_act && !gate_first;
    float v[PER], gv[PER], ss = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = threadIdx.x + 256 * j;
        v[j] = i < gs ? orow[i] : 0.f;
        gv[j] = 1.f;
        if (grow && gate_act && i < gs) {
            const float z = (float)grow[i];
            gv[j] = gate_act == 1 ? sigmoid_(z) : silu_(z);
        }
        if (pre) v[j] *= gv[j];
        ss += v[j] * v[j];
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float inv = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)gs + eps);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = threadIdx.x + 256 * j;
        if (i < gs) {
            float r = v[j] * inv * (weight ? ldf(weight, w_full ? (int64_t)g * gs + i : i) : 1.0f);
            if (post) r *= gv[j];
            y[t * y_stride + (int64_t)g * gs + i] = (A)r;
        }
    }
}

template <int DKQ, int SUBS, bool EXACT, bool PRE>
void launch_scan_pre(const ScanArgs& p, int64_t batch, hipStream_t st) {
    constexpr int COLS = 256 / SUBS;
    constexpr int CH = (3 * DKQ * SUBS + COLS + 4 + 255) / 256;
    constexpr int TOK = (32 / CH) < 2 ? 2 : (32 / CH);
    const unsigned colblocks = (unsigned)nvh_cdiv(p.dv, COLS);
    const size_t lds = sizeof(float) * (size_t)TOK * (((3 * p.dk + COLS + 4) & ~3) + COLS);
    if constexpr (EXACT) {
        if (p.nseg > 1) {
            const dim3 grid((unsigned)batch, (unsigned)p.H, colblocks * (unsigned)p.nseg);
            gated_linear_scan_kernel<DKQ, SUBS, EXACT, 1, PRE><<<grid, 256, lds, st>>>(p);
            gated_linear_scan_kernel<DKQ, SUBS, EXACT, 2, PRE><<<grid, 256, lds, st>>>(p);
            return;
        }
    }
    gated_linear_scan_kernel<DKQ, SUBS, EXACT, 0, PRE><<<dim3((unsigned)batch, (unsigned)p.H, colblocks), 256, lds, st>>>(p);
}

template <int DKQ, int SUBS, bool EXACT>
void launch_scan_as(const ScanArgs& p, int64_t batch, int read_first, hipStream_t st) {
    if (read_first) launch_scan_pre<DKQ, SUBS, EXACT, true>(p, batch, st);
    else launch_scan_pre<DKQ, SUBS, EXACT, false>(p, batch, st);
}

}  // namespace

extern "C" int32_t nvh_hgrn2_prep(const void* q, int64_t q_stride, const void* f, int64_t f_stride, const void* v, int64_t v_stride,
                                  const void* f_bias, const void* lower, float* out_q, float* out_k, float* out_w, float* out_v,
                                  int64_t num_tokens, int64_t n_k, int64_t n_v, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(q && f && v && f_bias && lower && out_q && out_k && out_w && out_v, NVH_EINVAL, "nvh_hgrn2_prep: null pointer");
    NVH_REQUIRE(num_tokens >= 0 && n_k > 0 && n_v > 0, NVH_EINVAL, "nvh_hgrn2_prep: bad sizes");
    if (num_tokens == 0) return NVH_OK;
    const Hgrn2PrepArgs p{q, f, v, q_stride, f_stride, v_stride, f_bias, lower, out_q, out_k, out_w, out_v, n_k, n_v};
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) hgrn2_prep_kernel<float><<<dim3((unsigned)num_tokens), 256, 0, st>>>(p);
    else hgrn2_prep_kernel<bf16><<<dim3((unsigned)num_tokens), 256, 0, st>>>(p);
    NVH_CHECK_LAUNCH("nvh_hgrn2_prep");
    return NVH_OK;
}

extern "C" int32_t nvh_gla_prep(const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v, int64_t v_stride,
                                const float* decay_logits, int64_t z_stride, float q_scale, float tau, float* out_q, float* out_k,
                                float* out_w, float* out_v, int64_t num_tokens, int64_t n_k, int64_t n_v, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(q && k && v && decay_logits && out_q && out_k && out_w && out_v, NVH_EINVAL, "nvh_gla_prep: null pointer");
    NVH_REQUIRE(num_tokens >= 0 && n_k > 0 && n_v > 0 && tau > 0.f, NVH_EINVAL, "nvh_gla_prep: bad sizes");
    if (num_tokens == 0) return NVH_OK;
    const GlaPrepArgs p{q, k, v, q_stride, k_stride, v_stride, decay_logits, z_stride, q_scale, 1.0f / tau, out_q, out_k, out_w, out_v, n_k, n_v};
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) gla_prep_kernel<float><<<dim3((unsigned)num_tokens), 256, 0, st>>>(p);
    else gla_prep_kernel<bf16><<<dim3((unsigned)num_tokens), 256, 0, st>>>(p);
    NVH_CHECK_LAUNCH("nvh_gla_prep");
    return NVH_OK;
}

extern "C" int32_t nvh_wkv_prep(const void* r, int64_t r_stride, const void* k, int64_t k_stride, const void* v, int64_t v_stride, const void* lowrank,
                                int64_t lowrank_stride, const void* w2, const void* w0, float* out_q, float* out_k, float* out_w, float* out_v,
                                int64_t num_tokens, int64_t n_k, int64_t n_v, int64_t rank, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(r && k && v && lowrank && w2 && w0 && out_q && out_k && out_w && out_v, NVH_EINVAL, "nvh_wkv_prep: null pointer");
    NVH_REQUIRE(num_tokens >= 0 && n_k > 0 && n_v > 0 && rank > 0 && rank <= 8192 && lowrank_stride >= rank, NVH_EINVAL, "nvh_wkv_prep: bad sizes");
    if (num_tokens == 0) return NVH_OK;
    const WkvPrepArgs p{r, k, v, lowrank, r_stride, k_stride, v_stride, lowrank_stride, w2, w0, out_q, out_k, out_w, out_v, n_k, n_v, (int)rank};
    hipStream_t st = (hipStream_t)stream;
    const size_t lds = sizeof(float) * (size_t)rank;
    if (act_f32) wkv_prep_kernel<float><<<dim3((unsigned)num_tokens), 256, lds, st>>>(p);
    else wkv_prep_kernel<bf16><<<dim3((unsigned)num_tokens), 256, lds, st>>>(p);
    NVH_CHECK_LAUNCH("nvh_wkv_prep");
    return NVH_OK;
}

extern "C" int32_t nvh_token_shift_mix(const void* h, int64_t h_stride, const float* state, const int32_t* slots, const int32_t* cu_seqlens_q,
                                       const int32_t* context_lens, int64_t batch, const void* mu, void* out, int64_t num_tokens, int64_t num_mixes,
                                       int64_t dim, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(h && state && slots && context_lens && mu && out, NVH_EINVAL, "nvh_token_shift_mix: null pointer");
    NVH_REQUIRE(batch >= 0 && num_tokens >= 0 && num_mixes > 0 && dim > 0 && h_stride >= dim && (cu_seqlens_q || num_tokens == batch), NVH_EINVAL,
                "nvh_token_shift_mix: bad sizes");
    if (num_tokens == 0 || batch == 0) return NVH_OK;
    const ShiftArgs p{h, h_stride, state, slots, cu_seqlens_q, context_lens, (int)batch, mu, out, num_tokens, (int)num_mixes, (int)dim,
                      (int)(dim % 8 == 0 && h_stride % 8 == 0 && nvh_aligned16(h) && nvh_aligned16(state) && nvh_aligned16(mu) && nvh_aligned16(out))};
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) token_shift_mix_kernel<float><<<dim3((unsigned)num_tokens), 256, 0, st>>>(p);
    else token_shift_mix_kernel<bf16><<<dim3((unsigned)num_tokens), 256, 0, st>>>(p);
    NVH_CHECK_LAUNCH("nvh_token_shift_mix");
    return NVH_OK;
}

extern "C" int32_t nvh_rotary_qkv_prep(const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v, int64_t v_stride,
                                       const int64_t* positions, const float* freq, float mag, int64_t rot_dims, int32_t interleaved, float q_scale,
                                       float k_scale, float* out_q, float* out_k, float* out_v, int64_t num_tokens, int64_t heads, int64_t dim,
                                       int64_t vdim, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(q && k && v && positions && out_q && out_k && out_v, NVH_EINVAL, "nvh_rotary_qkv_prep: null pointer");
    NVH_REQUIRE(num_tokens >= 0 && heads > 0 && dim > 0 && vdim > 0 && rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0 && (rot_dims == 0 || freq),
                NVH_EINVAL, "nvh_rotary_qkv_prep: bad sizes");
    if (num_tokens == 0) return NVH_OK;
    const RotPrepArgs a{q, k, v, q_stride, k_stride, v_stride, positions, freq, mag, q_scale, k_scale, (int)rot_dims, interleaved, (int)heads, (int)dim,
                        (int)vdim, out_q, out_k, out_v};
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) rotary_qkv_prep_kernel<float><<<dim3((unsigned)num_tokens), 256, 0, st>>>(a);
    else rotary_qkv_prep_kernel<bf16><<<dim3((unsigned)num_tokens), 256, 0, st>>>(a);
    NVH_CHECK_LAUNCH("nvh_rotary_qkv_prep");
    return NVH_OK;
}

static int32_t ssd_args(SsdPrepArgs& p, const void* xbc, int64_t xbc_stride, const void* dt, int64_t dt_stride, const void* conv_w, const void* conv_b,
                        const void* dt_bias, const void* a_log, float* conv_state, const int32_t* slots, const int32_t* cu_seqlens_q,
                        const int32_t* context_lens, int64_t batch, int64_t taps, int64_t heads, int64_t inner, int64_t gn) {
    NVH_REQUIRE(xbc && conv_w && slots && context_lens && (taps == 1 || conv_state), NVH_EINVAL, "ssd convolution: null pointer");
    NVH_REQUIRE(batch >= 0 && taps >= 1 && taps <= 64 && heads > 0 && inner > 0 && gn > 0 && xbc_stride >= inner + 2 * gn, NVH_EINVAL, "ssd convolution: bad sizes");
    p = SsdPrepArgs{xbc, xbc_stride, dt, dt_stride, conv_w, conv_b, dt_bias, a_log, conv_state, slots, cu_seqlens_q, context_lens,
                    (int)batch, (int)taps, (int)heads, (int)inner, (int)gn, nullptr, nullptr, nullptr, nullptr, nullptr};
    return NVH_OK;
}

extern "C" int32_t nvh_ssd_conv_prep(const void* xbc, int64_t xbc_stride, const void* dt, int64_t dt_stride, const void* conv_w, const void* conv_b,
                                     const void* dt_bias, const void* a_log, float* conv_state, const int32_t* slots, const int32_t* cu_seqlens_q,
                                     const int32_t* context_lens, int64_t batch, int64_t num_tokens, int64_t taps, int64_t heads, int64_t inner,
                                     int64_t gn, float* out_x, float* out_b, float* out_c, float* out_dt, float* out_decay, int32_t act_f32,
                                     nvh_stream_t stream) {
    SsdPrepArgs p;
    const int32_t rc = ssd_args(p, xbc, xbc_stride, dt, dt_stride, conv_w, conv_b, dt_bias, a_log, conv_state, slots, cu_seqlens_q, context_lens, batch, taps, heads, inner, gn);
    if (rc != NVH_OK) return rc;
    NVH_REQUIRE(dt && dt_bias && a_log && out_x && out_b && out_c && out_dt && out_decay && num_tokens >= 0, NVH_EINVAL, "nvh_ssd_conv_prep: null pointer");
    NVH_REQUIRE(cu_seqlens_q || num_tokens == batch, NVH_EINVAL, "nvh_ssd_conv_prep: one token per sequence without cu_seqlens_q");
    if (num_tokens == 0 || batch == 0) return NVH_OK;
    p.ov = out_x, p.ok = out_b, p.oq = out_c, p.oc = out_dt, p.ow = out_decay;
    hipStream_t st = (hipStream_t)stream;
    // few tokens: the channels are spread over more workgroups (a token's row is short work for one)
    const int64_t esz = act_f32 ? 4 : 2, per_lane = 16 / esz;            // elements per 16 bytes
    const bool vec = taps >= 2 && taps <= 4 && inner % 8 == 0 && gn % 8 == 0 && xbc_stride % per_lane == 0 && nvh_aligned16(xbc) && nvh_aligned16(conv_w) &&
                     (!conv_b || nvh_aligned16(conv_b)) && nvh_aligned16(conv_state) && nvh_aligned16(out_x) && nvh_aligned16(out_b) && nvh_aligned16(out_c);
    const int64_t lanes = vec ? (inner + 2 * gn) / 8 : inner + 2 * gn;
    const dim3 grid((unsigned)num_tokens, (unsigned)(num_tokens >= 512 ? 1 : std::min<int64_t>(nvh_cdiv(lanes, 256), 16)));
    if (vec) {
#define NVH_CONV_VEC(TAPS)                                                        \
    if (act_f32) ssd_conv_prep_vec_kernel<float, TAPS><<<grid, 256, 0, st>>>(p); \
    else ssd_conv_prep_vec_kernel<bf16, TAPS><<<grid, 256, 0, st>>>(p)
        if (taps == 2) { NVH_CONV_VEC(2); }
        else if (taps == 3) { NVH_CONV_VEC(3); }
        else { NVH_CONV_VEC(4); }
#undef NVH_CONV_VEC
    } else if (act_f32) {
        ssd_conv_prep_kernel<float><<<grid, 256, 0, st>>>(p);
    } else {
        ssd_conv_prep_kernel<bf16><<<grid, 256, 0, st>>>(p);
    }
    NVH_CHECK_LAUNCH("nvh_ssd_conv_prep");
    return NVH_OK;
}

extern "C" int32_t nvh_conv_state_update(const void* xbc, int64_t xbc_stride, float* conv_state, const int32_t* slots, const int32_t* cu_seqlens_q,
                                         const int32_t* context_lens, int64_t batch, int64_t taps, int64_t channels, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(xbc && slots && context_lens && batch >= 0 && taps >= 1 && channels > 0 && xbc_stride >= channels, NVH_EINVAL, "nvh_conv_state_update: bad argument");
    if (batch == 0 || taps == 1) return NVH_OK;
    NVH_REQUIRE(conv_state, NVH_EINVAL, "nvh_conv_state_update: null state");
    SsdPrepArgs p{};
    p.xbc = xbc, p.xbc_stride = xbc_stride, p.conv_state = conv_state, p.slots = slots, p.cu_seqlens_q = cu_seqlens_q, p.context_lens = context_lens;
    p.batch = (int)batch, p.taps = (int)taps, p.inner = (int)channels, p.gn = 0;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)batch, (unsigned)nvh_cdiv(channels, 256));
    if (act_f32) conv_state_update_kernel<float><<<grid, 256, 0, st>>>(p);
    else conv_state_update_kernel<bf16><<<grid, 256, 0, st>>>(p);
    NVH_CHECK_LAUNCH("nvh_conv_state_update");
    return NVH_OK;
}

extern "C" int32_t nvh_stream_conv(const float* x, const void* w, const float* state, const int32_t* slots, const int32_t* cu_seqlens_q,
                                   const int32_t* context_lens, void* h, int64_t h_stride, int64_t batch, int64_t num_tokens, int64_t taps, int64_t dim,
                                   int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(x && w && slots && context_lens && h && batch >= 0 && num_tokens >= 0 && taps >= 1 && dim > 0 && h_stride >= dim, NVH_EINVAL,
                "nvh_stream_conv: bad argument");
    NVH_REQUIRE(taps == 1 || state, NVH_EINVAL, "nvh_stream_conv: null state");
    NVH_REQUIRE(cu_seqlens_q || num_tokens == batch, NVH_EINVAL, "nvh_stream_conv: one token per sequence without cu_seqlens_q");
    if (num_tokens == 0 || batch == 0) return NVH_OK;
    const StreamConvArgs p{x, w, state, slots, cu_seqlens_q, context_lens, h, h_stride, (int)batch, (int)taps, (int)dim};
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)num_tokens, (unsigned)(num_tokens >= 512 ? 1 : std::min<int64_t>(nvh_cdiv(dim, 256), 16)));
    if (act_f32) stream_conv_kernel<float><<<grid, 256, 0, st>>>(p);
    else stream_conv_kernel<bf16><<<grid, 256, 0, st>>>(p);
    NVH_CHECK_LAUNCH("nvh_stream_conv");
    return NVH_OK;
}

// Key sizes whose scan has the segmented form (the exact instantiations below).
extern "C" int32_t nvh_scan_segmentable(int64_t dk) {
    return dk % 16 == 0 && (dk / 16 <= 4 || dk / 16 == 6 || dk / 16 == 8 || dk / 16 == 16);
}

extern "C" int32_t nvh_gated_linear_scan(const float* q, int64_t q_stride, const float* k, int64_t k_stride, int64_t qk_groups, const float* w,
                                         int64_t w_stride, int32_t w_scalar, const float* kscale, int64_t kscale_stride, const float* v,
                                         int64_t v_stride, const float* skip, float* state, const int32_t* slots, const int32_t* cu_seqlens_q,
                                         const int32_t* context_lens, float* out, int64_t batch, int64_t heads, int64_t dk, int64_t dv,
                                         int64_t segments, int64_t segment_min_tokens, float* ws_states, float* ws_decays, int32_t read_first,
                                         const float* bonus, nvh_stream_t stream) {
    NVH_REQUIRE(q && k && w && v && state && slots && context_lens && out, NVH_EINVAL, "nvh_gated_linear_scan: null pointer");
    NVH_REQUIRE(batch >= 0 && heads > 0 && dk > 0 && dv > 0 && qk_groups > 0 && heads % qk_groups == 0, NVH_EINVAL, "nvh_gated_linear_scan: bad sizes");
    NVH_REQUIRE(dk <= 512, NVH_ENOSYS, "nvh_gated_linear_scan: key size %ld above 512", (long)dk);
    if (batch == 0) return NVH_OK;
    ScanArgs p{q, k, q_stride, k_stride, (int)qk_groups, w, w_stride, w_scalar, kscale, kscale_stride, v, v_stride, skip, state, slots,
                     cu_seqlens_q, context_lens, out, (int)heads, (int)dk, (int)dv, 1, 1 << 30, ws_states, ws_decays, bonus};
    NVH_REQUIRE(read_first || !bonus, NVH_EINVAL, "nvh_gated_linear_scan: a bonus needs read_first");
    if (segments > 1 && nvh_scan_segmentable(dk)) {
        NVH_REQUIRE(segments <= 64 && segment_min_tokens >= 2 * segments && ws_states && ws_decays && cu_seqlens_q, NVH_EINVAL, "nvh_gated_linear_scan: bad segments");
        p.nseg = (int)segments;
        p.seg_min = (int)segment_min_tokens;
    }
    hipStream_t st = (hipStream_t)stream;
    // (the choice depends on dk alone, so a sequence sees one summation order whatever the batch or the cut)
    if (dk % 16 == 0) {
        switch (dk / 16) {
            case 1: launch_scan_as<1, 16, true>(p, batch, read_first, st); break;
            case 2: launch_scan_as<2, 16, true>(p, batch, read_first, st); break;
            case 3: launch_scan_as<3, 16, true>(p, batch, read_first, st); break;
            case 4: launch_scan_as<4, 16, true>(p, batch, read_first, st); break;
            case 6: launch_scan_as<6, 16, true>(p, batch, read_first, st); break;
            case 8: launch_scan_as<8, 16, true>(p, batch, read_first, st); break;
            case 16: launch_scan_as<16, 16, true>(p, batch, read_first, st); break;
            default:
                if (dk / 16 <= 8) launch_scan_as<8, 16, false>(p, batch, read_first, st);
                else if (dk / 16 <= 16) launch_scan_as<16, 16, false>(p, batch, read_first, st);
                else launch_scan_as<32, 16, false>(p, batch, read_first, st);
        }
    } else {
        const int dkq = (int)(dk + 3) / 4;
        if (dkq <= 8) launch_scan_as<8, 4, false>(p, batch, read_first, st);
        else if (dkq <= 16) launch_scan_as<16, 4, false>(p, batch, read_first, st);
        else if (dkq <= 32) launch_scan_as<32, 4, false>(p, batch, read_first, st);
        else if (dkq <= 64) launch_scan_as<64, 4, false>(p, batch, read_first, st);
        else launch_scan_as<32, 16, false>(p, batch, read_first, st);
    }
    NVH_CHECK_LAUNCH("nvh_gated_linear_scan");
    return NVH_OK;
}

extern "C" int32_t nvh_group_rmsnorm_gate(const float* o, const void* weight, int32_t weight_full, const void* gate, int64_t gate_stride,
                                          int32_t gate_act, int32_t gate_first, void* y, int64_t y_stride, int64_t rows, int64_t groups,
                                          int64_t group_size, float eps, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(o && y && rows >= 0 && groups > 0 && group_size > 0 && gate_act >= 0 && gate_act <= 2 && (!gate_act || gate), NVH_EINVAL,
                "nvh_group_rmsnorm_gate: bad argument");
    if (rows == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    // (the form depends on the group size alone: a row sees one summation order whatever the batch or the cut)
    if (group_size > 256 && group_size <= 8192 && rows * groups < (1ll << 31)) {
        const dim3 grid((unsigned)(rows * groups));
#define NVH_GN_BLOCK(A, PER) group_rmsnorm_gate_block_kernel<A, PER><<<grid, 256, 0, st>>>(o, (const A*)weight, weight_full, (const A*)gate, gate_stride, gate_act, gate_first, (A*)y, y_stride, (int)groups, (int)group_size, eps)
        if (group_size <= 2048) {
            if (act_f32) NVH_GN_BLOCK(float, 8);
            else NVH_GN_BLOCK(bf16, 8);
        } else {
            if (act_f32) NVH_GN_BLOCK(float, 32);
            else NVH_GN_BLOCK(bf16, 32);
        }
#undef NVH_GN_BLOCK
        NVH_CHECK_LAUNCH("nvh_group_rmsnorm_gate");
        return NVH_OK;
    }
    const unsigned blocks = (unsigned)nvh_cdiv(rows * groups, 4);
    if (act_f32) group_rmsnorm_gate_kernel<float><<<dim3(blocks), 256, 0, st>>>(o, (const float*)weight, weight_full, (const float*)gate, gate_stride, gate_act, gate_first, (float*)y, y_stride, rows, (int)groups, (int)group_size, eps);
    else group_rmsnorm_gate_kernel<bf16><<<dim3(blocks), 256, 0, st>>>(o, (const bf16*)weight, weight_full, (const bf16*)gate, gate_stride, gate_act, gate_first, (bf16*)y, y_stride, rows, (int)groups, (int)group_size, eps);
    NVH_CHECK_LAUNCH("nvh_group_rmsnorm_gate");
    return NVH_OK;
}
