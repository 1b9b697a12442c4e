// Generalized delta rule: a per-head matrix state S [dk, dv] in fp32 that every token updates,
//   S <- diag(w) S - (a * u) (u^T S) + k v^T     (both terms read the old S),   o = S^T r,
// with a decay w in (0, 1) and a removal rate a per key channel and u the unit-length key.
//   nvh_delta_prep   per token and channel, all in fp32: the decay from its low-rank logit
//                    w = exp(-c * sigmoid(w0 + W2 tanh(l))) (c = e^-1/2 by default), a = sigmoid(a_raw + a_bias),
//                    u = k / sqrt(sum k^2 + 1e-6); leaves, per token and head, the contiguous fp32 row
//                    [r | k | w | u | a*u | v] that the scan reads.
//   nvh_delta_scan   walks a sequence's tokens in order from the state its slot holds (or from zero when the sequence
//                    starts) and leaves the state there.  Columns of S are independent of each other, so the work is
//                    spread over (sequence, head, column); each column is held by 16 lanes (4 when dk is no multiple
//                    of 16), each with every 16th (4th) row, which meet twice per token in a cross-lane sum.  The order of every sum is fixed by the sizes alone: decoding
//                    token by token, in portions or in one piece gives the same bits.
//   nvh_delta_post   per head: o / rms(o), times the norm weight and the sigmoid output gate, to the activation type.
//   nvh_gated_delta_prep   the gated delta rule, S <- g S; d = beta (v - S^T k); S <- S + k d^T; o = S^T q, with one decay g per head
//                    and a write strength beta per head, is the recurrence above with w = g on every channel, u = k (a unit
//                    vector), a u = beta g k and the written key beta k: g S - beta g k (k^T S) + beta k v^T.  The prep runs the
//                    short causal convolution (continued from the sequence's carried inputs) and silu over the q | k | v
//                    channels, makes q and k unit vectors per head (q also times dk^-1/2), forms beta = sigmoid(b) and
//                    g = exp(-exp(A_log) softplus(a + dt_bias)), all in fp32, and leaves the scan's rows; q and k heads
//                    may be shared by groups of value heads, and the value size is free.
#include "common.h"

namespace {

template <typename A>
__device__ __forceinline__ float ldf(const A* p, int64_t i) {
    return (float)p[i];
}
__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

struct DeltaPrepArgs {
    const void *r, *k, *v;     // [T, ld] rows of H*dk
    int64_t r_stride, k_stride, v_stride;
    const void* a_raw;         // [T, ld]
    int64_t a_stride;
    const void* lowrank;       // [T, ld] rows of `rank` (the first decay projection, before its tanh)
    int64_t l_stride;
    const void *w2, *w0, *a_bias;   // [H*dk, rank], [H*dk], [H*dk]
    float* out;                // [T, H, 6, dk]: r | k | w | u | a*u | v per head, contiguous
    int H, dk, rank;
    float decay_scale;
};

struct GatedDeltaPrepArgs {
    const void* qkv;           // [T, ld]: the convolved channels q (G dk) | k (G dk) | v (H dv) of the projection row
    int64_t qkv_stride;
    const void *b, *a;         // [T, ld]: H columns each (write strength and decay logits)
    int64_t b_stride, a_stride;
    const void* conv_w;        // [C, taps], last column on the current token
    const void *dt_bias, *a_log;    // [H]
    const float* conv_state;   // [slots, taps - 1, C]
    const int32_t *slots, *cu_seqlens_q, *context_lens;
    float* out;                // [T, H, 5 dk + dv]: q | beta k | g | k | beta g k | v
    int batch, taps, H, G, dk, dv;
};

__device__ __forceinline__ float softplusf_(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// One workgroup per (token, value head): the convolved, activated channels of the head's q / k group and of its own v meet in LDS,
// two waves sum the squares of q and k, then the head's row is written.  (Heads that share a q / k group convolve it again each: a
// few hundred channels, against a launch that would otherwise have as many workgroups as tokens only.)
template <typename A>
__global__ __launch_bounds__(256) void gated_delta_prep_kernel(GatedDeltaPrepArgs p) {
    extern __shared__ float sh[];                            // [dk] q, [dk] k, [dv] v of this head, then the two inverse lengths
    const int64_t t = blockIdx.x;
    const int h = blockIdx.y, dk = p.dk, dv = p.dv, g = h / (p.H / p.G);
    const int nqk = p.G * dk, C = 2 * nqk + p.H * dv, taps = p.taps, n = 2 * dk + dv;
    float* inv = sh + n;
    int seq = (int)t;
    if (p.cu_seqlens_q) {
        int lo_b = 0, hi_b = p.batch;                        // the sequence whose rows hold token t
        while (hi_b - lo_b > 1) {
            const int mid = (lo_b + hi_b) >> 1;
            if (p.cu_seqlens_q[mid] <= t) lo_b = mid;
            else hi_b = mid;
        }
        seq = lo_b;
    }
    const int lo = p.cu_seqlens_q ? p.cu_seqlens_q[seq] : seq, hi = p.cu_seqlens_q ? p.cu_seqlens_q[seq + 1] : seq + 1;
    const int j = (int)t - lo;
    const int slot = p.slots[seq];
    const bool carried = slot >= 0 && p.context_lens[seq] != hi - lo;
    const float* st = carried ? p.conv_state + (int64_t)slot * (taps - 1) * C : nullptr;
    for (int e = threadIdx.x; e < n; e += 256) {
        const int c = e < dk ? g * dk + e : (e < 2 * dk ? nqk + g * dk + (e - dk) : 2 * nqk + h * dv + (e - 2 * dk));      // the channel of the row
        float acc = 0.f;
        for (int k = 0; k < taps; ++k) {                     // tap k multiplies the input taps - 1 - k tokens back
            const int back = taps - 1 - k, src = j - back;
            float in = 0.f;
            if (src >= 0) in = ldf((const A*)p.qkv, (t - back) * p.qkv_stride + c);
            else if (st) in = st[(int64_t)(taps - 1 + src) * C + c];
            acc = __builtin_fmaf(ldf((const A*)p.conv_w, (int64_t)c * taps + k), in, acc);
        }
        sh[e] = acc / (1.0f + expf(-acc));
    }
    const float beta = sigmoidf_(ldf((const A*)p.b, t * p.b_stride + h));
    const float dec = expf(-expf(ldf((const A*)p.a_log, h)) * softplusf_(ldf((const A*)p.a, t * p.a_stride + h) + ldf((const A*)p.dt_bias, h)));
    __syncthreads();
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (wave < 2) {                                          // q, k
        float ss = 0.f;
        for (int i = lane; i < dk; i += 64) ss += sh[wave * dk + i] * sh[wave * dk + i];
        ss = wave_sum(ss);
        if (lane == 0) inv[wave] = 1.0f / sqrtf(ss + 1e-6f);
    }
    __syncthreads();
    const int row = 5 * dk + dv;
    const float qs = inv[0] / sqrtf((float)dk), ks = inv[1];
    float* out = p.out + (t * p.H + h) * (int64_t)row;
    for (int i = threadIdx.x; i < dk; i += 256) {
        const float ku = sh[dk + i] * ks;
        out[i] = sh[i] * qs;
        out[dk + i] = beta * ku;
        out[2 * dk + i] = dec;
        out[3 * dk + i] = ku;
        out[4 * dk + i] = beta * dec * ku;
    }
    for (int i = threadIdx.x; i < dv; i += 256) out[5 * dk + i] = sh[2 * dk + i];
}

template <typename A>
__global__ __launch_bounds__(256) void delta_prep_kernel(DeltaPrepArgs p) {
    extern __shared__ float tl[];                            // tanh of the low-rank row
    const int64_t t = blockIdx.x;
    for (int r = threadIdx.x; r < p.rank; r += 256) tl[r] = tanhf(ldf((const A*)p.lowrank, t * p.l_stride + r));
    __syncthreads();
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, dk = p.dk;
    for (int h = blockIdx.y * 4 + wave; h < p.H; h += 4 * gridDim.y) {      // one head per wave; grid.y covers the heads four at a time
        float* out = p.out + (t * p.H + h) * 6 * dk;
        float ss = 0.f;
        for (int i = lane; i < dk; i += 64) {
            const float kv = ldf((const A*)p.k, t * p.k_stride + h * dk + i);
            ss += kv * kv;
        }
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss + 1e-6f);
        for (int i = lane; i < dk; i += 64) {
            const int c = h * dk + i;
            float z = ldf((const A*)p.w0, c);
            const A* w2r = (const A*)p.w2 + (int64_t)c * p.rank;
            for (int r = 0; r < p.rank; ++r) z = __builtin_fmaf(ldf(w2r, r), tl[r], z);
            const float kv = ldf((const A*)p.k, t * p.k_stride + c);
            const float u = kv * inv;
            const float a = sigmoidf_(ldf((const A*)p.a_raw, t * p.a_stride + c) + ldf((const A*)p.a_bias, c));
            out[i] = ldf((const A*)p.r, t * p.r_stride + c);
            out[dk + i] = kv;
            out[2 * dk + i] = expf(-p.decay_scale * sigmoidf_(z));
            out[3 * dk + i] = u;
            out[4 * dk + i] = a * u;
            out[5 * dk + i] = ldf((const A*)p.v, t * p.v_stride + c);
        }
    }
}

struct DeltaScanArgs {
    const float* pack;         // [T, H, 5 dk + dv]: r | k | w | u | a*u (dk each) | v (dv) per head, from a prep kernel
    float* state;              // [slots, H, dk, dv]
    const int32_t* slots;      // [B]
    const int32_t* cu_seqlens_q;    // [B+1] or null (one token per sequence)
    const int32_t* context_lens;    // [B]: tokens of the sequence including this step's (a step that holds them all starts from zero)
    float* out;                // [T, H*dv]
    int H, dk, dv;
};

// Lanes per state column (SUBS: 16 when dk is a multiple of 16, else 4), rows i = SUBS * ii + sub held by lane `sub`; a
// workgroup of 256 lanes owns 256 / SUBS columns of one (sequence, head).  Tokens are staged TOK at a time: the loads
// of the next TOK tokens are in flight (in registers) while the current ones are walked from LDS.
// EXACT: dk == DKQ * SUBS, so the loops over a lane's rows carry no run-time bound (see attention_any.hip).
template <int DKQ, int SUBS, bool EXACT>
__global__ __launch_bounds__(256) void delta_scan_kernel(DeltaScanArgs p) {
    constexpr int COLS = 256 / SUBS;
    constexpr int CH = (5 * DKQ * SUBS + COLS + 255) / 256;  // loads per lane and token
    constexpr int TOK = (32 / CH) < 2 ? 2 : (32 / CH);
    extern __shared__ float sm[];                            // [TOK][5 dk + COLS]: r | k | w | u | au | v (this workgroup's columns)
    const int seq = blockIdx.x, head = blockIdx.y;
    const int dk = p.dk, dv = p.dv, dkq = (dk + SUBS - 1) / SUBS;      // rows i = SUBS * ii + sub >= dk (ragged dk) are held as zeros
    const int col0 = blockIdx.z * COLS, lcol = threadIdx.x / SUBS, col = col0 + lcol, sub = threadIdx.x % SUBS;
    const bool live = col < dv;
    const int lo = p.cu_seqlens_q ? p.cu_seqlens_q[seq] : seq, hi = p.cu_seqlens_q ? p.cu_seqlens_q[seq + 1] : seq + 1;
    const int slot = p.slots[seq];
    if (slot < 0 || hi <= lo) return;                        // a padded row (uniform over the workgroup)
    const bool fresh = p.context_lens[seq] == hi - lo;
    float* sp = p.state + (((int64_t)slot * p.H + head) * dk) * dv;
    float S[DKQ];
    // rows of a lane: DKQ consecutive ones when the sizes are exact (one 16-byte LDS read per operand and four rows), every
    // SUBS-th one otherwise
    auto row_of = [&](int ii) { return EXACT ? DKQ * sub + ii : SUBS * ii + sub; };
#pragma unroll
    for (int ii = 0; ii < DKQ; ++ii) S[ii] = (live && !fresh && (EXACT || row_of(ii) < dk)) ? sp[(int64_t)row_of(ii) * dv + col] : 0.f;
    const int rowf = 5 * dk + COLS;
    // Row of a token as this workgroup needs it: the five dk-vectors, then its COLS columns of v.  Every load is
    // unconditional (indices clamped into the row and into the sequence), so all of a stage's loads are in flight together.
    float pre[TOK][CH];
    const int prow = 5 * dk + dv;                            // a head's row of the pack
    const float* base = p.pack + (int64_t)head * prow;
    const int64_t tok_stride = (int64_t)p.H * prow;
    auto fetch = [&](int t0) {
#pragma unroll
        for (int tt = 0; tt < TOK; ++tt) {
            const int64_t tok = min(t0 + tt, hi - 1);
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int e = threadIdx.x + 256 * c;
                const int src = min(e < 5 * dk ? e : e + col0, prow - 1);
                pre[tt][c] = base[tok * tok_stride + src];
            }
        }
    };
    fetch(lo);
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
        // A token's operands are read from LDS one token ahead, so the reads' latency is off the chain S -> dot -> S.
        float cr[DKQ], ck[DKQ], cw[DKQ], cu[DKQ], ca[DKQ], cv;
        auto read_token = [&](int tt, float (&xr)[DKQ], float (&xk)[DKQ], float (&xw)[DKQ], float (&xu)[DKQ], float (&xa)[DKQ], float& xv) {
            const float* row = sm + tt * rowf;
            if constexpr (EXACT && DKQ % 4 == 0) {
#pragma unroll
                for (int c4 = 0; c4 < DKQ / 4; ++c4) {
                    const int i = DKQ * sub + 4 * c4;
                    const f32x4 vr = *reinterpret_cast<const f32x4*>(row + i), vk = *reinterpret_cast<const f32x4*>(row + dk + i),
                                vw = *reinterpret_cast<const f32x4*>(row + 2 * dk + i), vu = *reinterpret_cast<const f32x4*>(row + 3 * dk + i),
                                va = *reinterpret_cast<const f32x4*>(row + 4 * dk + i);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        xr[4 * c4 + e] = vr[e];
                        xk[4 * c4 + e] = vk[e];
                        xw[4 * c4 + e] = vw[e];
                        xu[4 * c4 + e] = vu[e];
                        xa[4 * c4 + e] = va[e];
                    }
                }
                xv = row[5 * dk + lcol];
                return;
            }
#pragma unroll
            for (int ii = 0; ii < DKQ; ++ii)
                if (EXACT || ii < dkq) {
                    const int i = row_of(ii);
                    const bool in = EXACT || i < dk;         // (a row beyond dk: all operands zero, its state stays zero)
                    xr[ii] = in ? row[i] : 0.f;
                    xk[ii] = in ? row[dk + i] : 0.f;
                    xw[ii] = in ? row[2 * dk + i] : 0.f;
                    xu[ii] = in ? row[3 * dk + i] : 0.f;
                    xa[ii] = in ? row[4 * dk + i] : 0.f;
                }
            xv = row[5 * dk + lcol];
        };
        // one token: reads S, leaves the new S and the output (the operands were read one token ahead)
        auto token = [&](int tt, const float (&xr)[DKQ], const float (&xk)[DKQ], const float (&xw)[DKQ], const float (&xu)[DKQ],
                         const float (&xa)[DKQ], float xv) {
            float dot = 0.f;
#pragma unroll
            for (int ii = 0; ii < DKQ; ++ii)
                if (EXACT || ii < dkq) dot = __builtin_fmaf(xu[ii], S[ii], dot);
            if constexpr (SUBS == 16) {
                dot = row16_sum(dot);
            } else {
                dot += NVH_DPP(dot, 0xB1);
                dot += NVH_DPP(dot, 0x4E);
            }
            float o = 0.f;
#pragma unroll
            for (int ii = 0; ii < DKQ; ++ii)
                if (EXACT || ii < dkq) {
                    const float sn = __builtin_fmaf(xw[ii], S[ii], __builtin_fmaf(xk[ii], xv, -(xa[ii] * dot)));
                    S[ii] = sn;
                    o = __builtin_fmaf(sn, xr[ii], o);
                }
            if constexpr (SUBS == 16) {
                o = row16_sum(o);
            } else {
                o += NVH_DPP(o, 0xB1);
                o += NVH_DPP(o, 0x4E);
            }
            if (live && sub == 0) p.out[(int64_t)(t0 + tt) * p.H * dv + head * dv + col] = o;
        };
        // two register sets take turns (no copies): while one token is worked on, the next one's operands arrive
        float nr[DKQ], nk[DKQ], nw[DKQ], nu[DKQ], na[DKQ], nv;
        read_token(0, cr, ck, cw, cu, ca, cv);
        int tt = 0;
        for (; tt + 1 < nt; tt += 2) {
            read_token(tt + 1, nr, nk, nw, nu, na, nv);
            token(tt, cr, ck, cw, cu, ca, cv);
            read_token(min(tt + 2, TOK - 1), cr, ck, cw, cu, ca, cv);
            token(tt + 1, nr, nk, nw, nu, na, nv);
        }
        if (tt < nt) token(tt, cr, ck, cw, cu, ca, cv);
    }
    if (live) {
#pragma unroll
        for (int ii = 0; ii < DKQ; ++ii)
            if (EXACT || row_of(ii) < dk) sp[(int64_t)row_of(ii) * dv + col] = S[ii];
    }
}

template <typename A>
__global__ __launch_bounds__(256) void delta_post_kernel(const float* __restrict__ o, const A* __restrict__ norm_w, const A* __restrict__ gate,
                                                         int64_t gate_stride, A* __restrict__ y, int64_t y_stride, int64_t rows, int H, int dv, float eps) {
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);     // (token, head) per wave
    if (item >= rows * H) return;
    const int64_t t = item / H;
    const int h = (int)(item - t * H), lane = threadIdx.x & 63;
    const float* orow = o + (t * H + h) * dv;
    float ss = 0.f;
    for (int i = lane; i < dv; i += 64) ss += orow[i] * orow[i];
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
    for (int i = lane; i < dv; i += 64) {
        const int c = h * dv + i;
        const float g = gate ? sigmoidf_(ldf(gate, t * gate_stride + c)) : 1.0f;
        y[t * y_stride + c] = (A)(orow[i] * inv * ldf(norm_w, c) * g);
    }
}

}  // namespace

extern "C" int32_t nvh_delta_prep(const void* r, int64_t r_stride, const void* k, int64_t k_stride, const void* v, int64_t v_stride,
                                  const void* a_raw, int64_t a_stride, const void* lowrank, int64_t lowrank_stride,
                                  const void* w2, const void* w0, const void* a_bias, float* out, int64_t num_tokens, int64_t heads, int64_t dk,
                                  int64_t rank, float decay_scale, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(r && k && v && a_raw && lowrank && w2 && w0 && a_bias && out, NVH_EINVAL, "nvh_delta_prep: null pointer");
    NVH_REQUIRE(num_tokens >= 0 && heads > 0 && dk > 0 && rank > 0 && rank <= 8192, NVH_EINVAL, "nvh_delta_prep: bad sizes");
    if (num_tokens == 0) return NVH_OK;
    DeltaPrepArgs p{r, k, v, r_stride, k_stride, v_stride, a_raw, a_stride, lowrank, lowrank_stride, w2, w0, a_bias, out, (int)heads, (int)dk, (int)rank, decay_scale};
    hipStream_t st = (hipStream_t)stream;
    const size_t lds = sizeof(float) * (size_t)rank;
    const dim3 grid((unsigned)num_tokens, (unsigned)nvh_cdiv(heads, 4));
    if (act_f32) delta_prep_kernel<float><<<grid, 256, lds, st>>>(p);
    else delta_prep_kernel<bf16><<<grid, 256, lds, st>>>(p);
    NVH_CHECK_LAUNCH("nvh_delta_prep");
    return NVH_OK;
}

template <int DKQ, int SUBS, bool EXACT>
static void launch_delta_scan_as(const DeltaScanArgs& p, int64_t batch, hipStream_t st) {
    constexpr int COLS = 256 / SUBS;
    constexpr int CH = (5 * DKQ * SUBS + COLS + 255) / 256;
    constexpr int TOK = (32 / CH) < 2 ? 2 : (32 / CH);
    const dim3 grid((unsigned)batch, (unsigned)p.H, (unsigned)nvh_cdiv(p.dv, COLS));
    const size_t lds = sizeof(float) * (size_t)TOK * (5 * p.dk + COLS);
    delta_scan_kernel<DKQ, SUBS, EXACT><<<grid, 256, lds, st>>>(p);
}

static int32_t launch_delta_scan(const DeltaScanArgs& p, int64_t batch, hipStream_t st) {
    // (the choice depends on dk alone, so a sequence sees one summation order whatever the batch or the cut)
    if (p.dk % 16 == 0) {
        switch (p.dk / 16) {
            case 1: launch_delta_scan_as<1, 16, true>(p, batch, st); break;
            case 2: launch_delta_scan_as<2, 16, true>(p, batch, st); break;
            case 3: launch_delta_scan_as<3, 16, true>(p, batch, st); break;
            case 4: launch_delta_scan_as<4, 16, true>(p, batch, st); break;
            case 6: launch_delta_scan_as<6, 16, true>(p, batch, st); break;
            case 8: launch_delta_scan_as<8, 16, true>(p, batch, st); break;
            case 16: launch_delta_scan_as<16, 16, true>(p, batch, st); break;
            default:
                if (p.dk / 16 <= 8) launch_delta_scan_as<8, 16, false>(p, batch, st);
                else launch_delta_scan_as<16, 16, false>(p, batch, st);
        }
    } else {
        const int dkq = (p.dk + 3) / 4;
        if (dkq <= 8) launch_delta_scan_as<8, 4, false>(p, batch, st);
        else if (dkq <= 16) launch_delta_scan_as<16, 4, false>(p, batch, st);
        else if (dkq <= 32) launch_delta_scan_as<32, 4, false>(p, batch, st);
        else launch_delta_scan_as<64, 4, false>(p, batch, st);
    }
    NVH_CHECK_LAUNCH("nvh_delta_scan");
    return NVH_OK;
}

extern "C" int32_t nvh_gated_delta_prep(const void* qkv, int64_t qkv_stride, const void* b, int64_t b_stride, const void* a, int64_t a_stride,
                                        const void* conv_w, const void* dt_bias, const void* a_log, const float* conv_state, const int32_t* slots,
                                        const int32_t* cu_seqlens_q, const int32_t* context_lens, float* out, int64_t batch, int64_t num_tokens,
                                        int64_t taps, int64_t heads, int64_t qk_heads, int64_t dk, int64_t dv, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(qkv && b && a && conv_w && dt_bias && a_log && slots && context_lens && out, NVH_EINVAL, "nvh_gated_delta_prep: null pointer");
    NVH_REQUIRE(batch >= 0 && num_tokens >= 0 && taps >= 1 && heads > 0 && qk_heads > 0 && heads % qk_heads == 0 && dk > 0 && dv > 0, NVH_EINVAL,
                "nvh_gated_delta_prep: bad sizes");
    NVH_REQUIRE(taps == 1 || conv_state, NVH_EINVAL, "nvh_gated_delta_prep: null state");
    NVH_REQUIRE(cu_seqlens_q || num_tokens == batch, NVH_EINVAL, "nvh_gated_delta_prep: one token per sequence without cu_seqlens_q");
    const int64_t channels = 2 * qk_heads * dk + heads * dv;
    NVH_REQUIRE(qkv_stride >= channels, NVH_EINVAL, "nvh_gated_delta_prep: projection row too short");
    const size_t lds = sizeof(float) * (size_t)(2 * dk + dv + 2);
    NVH_REQUIRE(lds <= 64 * 1024 && heads <= 65535, NVH_ENOSYS, "nvh_gated_delta_prep: head sizes %ld + %ld above the kernel's limit", (long)dk, (long)dv);
    if (num_tokens == 0 || batch == 0) return NVH_OK;
    GatedDeltaPrepArgs p{qkv, qkv_stride, b, a, b_stride, a_stride, conv_w, dt_bias, a_log, conv_state, slots, cu_seqlens_q, context_lens, out,
                         (int)batch, (int)taps, (int)heads, (int)qk_heads, (int)dk, (int)dv};
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)num_tokens, (unsigned)heads);
    if (act_f32) gated_delta_prep_kernel<float><<<grid, 256, lds, st>>>(p);
    else gated_delta_prep_kernel<bf16><<<grid, 256, lds, st>>>(p);
    NVH_CHECK_LAUNCH("nvh_gated_delta_prep");
    return NVH_OK;
}

extern "C" int32_t nvh_delta_scan(const float* pack, float* state, const int32_t* slots, const int32_t* cu_seqlens_q,
                                  const int32_t* context_lens, float* out, int64_t batch, int64_t heads, int64_t dk, int64_t dv, nvh_stream_t stream) {
    NVH_REQUIRE(pack && state && slots && context_lens && out, NVH_EINVAL, "nvh_delta_scan: null pointer");
    NVH_REQUIRE(batch >= 0 && heads > 0 && dk > 0 && dv > 0, NVH_EINVAL, "nvh_delta_scan: bad sizes");
    NVH_REQUIRE(dk <= 256, NVH_ENOSYS, "nvh_delta_scan: key size %ld above 256", (long)dk);
    if (batch == 0) return NVH_OK;
    DeltaScanArgs p{pack, state, slots, cu_seqlens_q, context_lens, out, (int)heads, (int)dk, (int)dv};
    return launch_delta_scan(p, batch, (hipStream_t)stream);
}

extern "C" int32_t nvh_delta_post(const float* o, const void* norm_weight, const void* gate, int64_t gate_stride, void* y, int64_t y_stride,
                                  int64_t rows, int64_t heads, int64_t dv, float eps, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(o && norm_weight && y && rows >= 0 && heads > 0 && dv > 0, NVH_EINVAL, "nvh_delta_post: bad argument");
    if (rows == 0) return NVH_OK;
    const unsigned blocks = (unsigned)nvh_cdiv(rows * heads, 4);
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) delta_post_kernel<float><<<dim3(blocks), 256, 0, st>>>(o, (const float*)norm_weight, (const float*)gate, gate_stride, (float*)y, y_stride, rows, (int)heads, (int)dv, eps);
    else delta_post_kernel<bf16><<<dim3(blocks), 256, 0, st>>>(o, (const bf16*)norm_weight, (const bf16*)gate, gate_stride, (bf16*)y, y_stride, rows, (int)heads, (int)dv, eps);
    NVH_CHECK_LAUNCH("nvh_delta_post");
    return NVH_OK;
}
