// Paged causal attention for any head sizes (query/key size `dim`, value size `vdim`, any page size), with the pieces a
// gated, value-rotating attention needs around it:
//   nvh_attn_rotary_prep  per token, over the fused projection row [q | k | v | gate]: RMS norm over the WHOLE q and the
//                         whole k projection, or over every head by itself with one weight row shared by the heads
//                         (norm_per_head), partial rotary on q and k (frequency table given by the
//                         caller, so any scaling rule fits), rotation of the value by its own position over all of
//                         vdim, sigmoid of the per-head gate; q goes to a packed buffer, k and v to their cache slots.
//                         Keys are cached [pages, page, G, dim]; values TRANSPOSED within a page, [pages, G, vdim, page],
//                         so the attention reads a value column over consecutive keys in one piece (its matrix
//                         product wants V^T) and never transposes on the fly.
//   nvh_attn_paged_any    softmax attention of var-len queries over the paged cache, scores / weights in fp32; the
//                         epilogue turns each head's output back by the query's position and multiplies the gate.
//                         Optional: a distance bias, score -= slope[head] * (query position - key position), and a
//                         sliding window that keeps the first tokens: query i sees key j <= i when i - j < window or
//                         j < keep_first; key tiles that no query of a workgroup can see are never loaded.
//                         Optional: chunks, query i sees key j <= i only when both lie in the same block of `chunk`
//                         positions counted from the sequence's start; and a sink per head, a learned logit that joins the
//                         softmax's denominator as one more term, as it is, standing for no token (it is the state a row starts from:
//                         maximum = sink, sum = 1, output = 0).
//                         Steps in which every sequence brings one query: the heads that share a KV head share a workgroup
//                         (groups of more than 16 heads in parts); when that leaves most of the chip idle, a sequence's key
//                         tiles are dealt out to several workgroups whose rows a second launch merges.
// Activations and caches are of type A (bf16 or fp32).  Key tiles always start at key 0 of a sequence and every query
// row keeps its own running maximum and sum, so a query's result does not depend on how the prompt was cut into steps
// or on what else is in the batch.
#include "common.h"

namespace {

template <typename A>
__device__ __forceinline__ float ldf(const A* p, int64_t i) {
    return (float)p[i];
}

__device__ __forceinline__ float block_sum_256(float v, float* scratch) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    return scratch[0] + scratch[1] + scratch[2] + scratch[3];
}

struct PrepArgs {
    const void* proj;          // [T, ld] : q (H*dim) | k (G*dim) | v (G*vdim) | gate (H)
    int64_t ld;
    const void *q_norm, *k_norm;   // [H*dim], [G*dim]; norm_per_head: [dim] each, shared by the heads
    int norm_per_head;
    float eps;
    const int64_t* positions;
    const float* qk_freq;      // [rot_dims / 2]
    float qk_mag;
    int rot_dims, qk_interleaved;
    const float* v_freq;       // [vdim / 2], or null: values are stored as they are
    int v_interleaved;
    void* q_out;               // [T, H*dim]
    float* gate_out;           // [T, H], or null (no gate columns in proj)
    void *k_cache, *v_cache;   // [pages, page, G, dim], [pages, G, vdim, page] (values transposed within a page)
    const int32_t* slot_mapping;
    int H, G, dim, vdim, page;
};

template <typename A>
__global__ __launch_bounds__(256) void attn_rotary_prep_kernel(PrepArgs a) {
    __shared__ float red[4];
    extern __shared__ float head_inv[];                      // norm_per_head: 1 / rms of every q head, then of every k head
    const int64_t t = blockIdx.x;
    const A* row = (const A*)a.proj + t * a.ld;
    const int nq = a.H * a.dim, nk = a.G * a.dim, nv = a.G * a.vdim;
    const A* qr = row;
    const A* kr = row + nq;
    const A* vr = kr + nk;
    float inv_q = 1.f, inv_k = 1.f;
    if (a.q_norm && a.norm_per_head) {                       // a wave per head in turn (q heads, then k heads: they lie one after the other)
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
        for (int h = wave; h < a.H + a.G; h += 4) {
            const A* hr = qr + (int64_t)h * a.dim;
            float ss = 0.f;
            for (int i = lane; i < a.dim; i += 64) {
                const float v = ldf(hr, i);
                ss += v * v;
            }
            ss = wave_sum(ss);
            if (lane == 0) head_inv[h] = 1.0f / sqrtf(ss / (float)a.dim + a.eps);
        }
        __syncthreads();
    } else if (a.q_norm) {                                   // (null norm weights: q and k pass as they are)
        float sq = 0.f, sk = 0.f;
        for (int i = threadIdx.x; i < nq; i += 256) {
            const float v = ldf(qr, i);
            sq += v * v;
        }
        for (int i = threadIdx.x; i < nk; i += 256) {
            const float v = ldf(kr, i);
            sk += v * v;
        }
        sq = block_sum_256(sq, red);
        sk = block_sum_256(sk, red);
        inv_q = 1.0f / sqrtf(sq / (float)nq + a.eps), inv_k = 1.0f / sqrtf(sk / (float)nk + a.eps);
    }
    const float pos = (float)a.positions[t];
    const int64_t slot = a.slot_mapping ? a.slot_mapping[t] : -1;
    // q and k: norm, then rotary on the first rot_dims dimensions of every head
    for (int which = 0; which < 2; ++which) {
        const int n = which ? nk : nq;
        const A* src = which ? kr : qr;
        const A* wn = (const A*)(which ? a.k_norm : a.q_norm);
        const float inv = which ? inv_k : inv_q;
        const int hbase = which ? a.H : 0;
        A* dst = which ? (slot >= 0 && a.k_cache ? (A*)a.k_cache + slot * nk : nullptr) : (A*)a.q_out + t * nq;
        if (!dst) continue;
        for (int i = threadIdx.x; i < n; i += 256) {
            const int d = i % a.dim;
            const float rinv = a.norm_per_head && wn ? head_inv[hbase + i / a.dim] : inv;
            float v = wn ? ldf(src, i) * rinv * ldf(wn, a.norm_per_head ? d : i) : ldf(src, i);
            if (d < a.rot_dims) {
                int partner, pair;
                bool first;
                pair_of(d, a.rot_dims, a.qk_interleaved, partner, pair, first);
                const int j = i - d + partner;
                const float o = wn ? ldf(src, j) * rinv * ldf(wn, a.norm_per_head ? partner : j) : ldf(src, j);
                float sn, cs;
                rot_sincos<A>(pos * a.qk_freq[pair], sn, cs);
                const float c = cs * a.qk_mag, s = sn * a.qk_mag;
                v = first ? v * c - o * s : v * c + o * s;
            }
            dst[i] = (A)v;
        }
    }
    if (slot >= 0 && a.v_cache) {
        A* dst = (A*)a.v_cache + (slot / a.page) * a.page * nv + slot % a.page;      // element i of the row goes to dst[i * page]
        for (int i = threadIdx.x; i < nv; i += 256) {
            float v = ldf(vr, i);
            if (a.v_freq) {
                const int d = i % a.vdim;
                int partner, pair;
                bool first;
                pair_of(d, a.vdim, a.v_interleaved, partner, pair, first);
                const float o = ldf(vr, i - d + partner);
                float s, c;
                rot_sincos<A>(pos * a.v_freq[pair], s, c);
                v = first ? v * c - o * s : v * c + o * s;
            }
            dst[(int64_t)i * a.page] = (A)v;
        }
    }
    if (a.gate_out)
        for (int h = threadIdx.x; h < a.H; h += 256) a.gate_out[t * a.H + h] = 1.0f / (1.0f + expf(-ldf(vr + nv, h)));
}

// ---------------------------------------------------------------------------------------------------------------
constexpr int AQ = 16;        // queries per workgroup (one 16-lane row of a wave per query)
constexpr int AK = 32;        // keys per tile
constexpr int AVC_MAX = 32;   // value columns per lane (the kernel's AVC: 16, or 32 for wide values): vdim <= 16 * AVC_MAX

struct AttnArgs {
    const void* q;             // [T, H*dim]
    const void *k_cache, *v_cache;
    const int32_t* cu_seqlens_q;    // [B+1], or null: one query per sequence (row b is sequence b)
    const int32_t* context_lens;    // [B]: keys of the sequence including this step's tokens
    const int32_t* block_tables;
    int64_t table_stride;
    int batch, page;
    int H, G, dim, vdim;
    float scale;
    const float* gate;         // [T, H] or null
    const float* v_freq;       // [vdim/2] or null: no turning back
    int v_interleaved;
    void* out;                 // [T, H*vdim]
    const float* slopes;       // [H] or null: score -= slopes[head] * (query position - key position)
    int window, keep_first;    // window > 0: key j is visible to query i only when i - j < window or j < keep_first
    int chunk;                 // chunk > 0: ... and only when j >= (i / chunk) * chunk
    const float* sinks;        // [H] or null: a logit per head that joins the denominator of every row of that head
    int pages_offset;          // byte offset in LDS of the sequence's page ids (matrix-core kernel)
    int ml_offset;             // ... and of the waves' (max, sum) pairs in the one-query form
    int kv_split;              // one-query form: workgroups per (sequence, KV head), each with H / (G kv_split) of the group's heads
    int key_parts;             // one-query form: workgroups that share a sequence's key tiles (tile j goes to part j % key_parts); > 1: the
    float* parts;              // parts leave [batch, G kv_split, key_parts, 16, vdim + 2] (unnormalised rows, then max and sum) here
};

// The key tiles (of `tile` keys, starting at multiples of it) that a workgroup whose first query sits at position qlo has to
// walk: all of them without a window; with one, the tiles that hold kept first tokens and then those from the window of
// the first query on.  next(k0) is the start of the tile after k0.
struct TileWalk {
    int first_end, win_start, tile;
    __device__ __forceinline__ TileWalk(int window, int keep_first, int chunk, int qlo, int tile_) : tile(tile_) {
        first_end = window > 0 ? ((keep_first + tile_ - 1) / tile_) * tile_ : 0;
        win_start = window > 0 ? (max(qlo - window + 1, 0) / tile_) * tile_ : 0;
        // (the chunk of the first query starts no later than any other query's: earlier tiles are seen by none)
        if (chunk > 0) win_start = max(win_start, ((qlo / chunk) * chunk / tile_) * tile_);
    }
    __device__ __forceinline__ int next(int k0) const {
        const int n = k0 + tile;
        return (n >= first_end && n < win_start) ? win_start : n;
    }
};

__device__ __forceinline__ bool key_visible(int key, int qpos, int window, int keep_first, int chunk) {
    return key <= qpos && (window <= 0 || qpos - key < window || key < keep_first) && (chunk <= 0 || key >= (qpos / chunk) * chunk);
}

template <typename A, int AVC>
__global__ __launch_bounds__(256) void attn_paged_any_kernel(AttnArgs a) {
    extern __shared__ float smem[];
    // which (sequence, query tile) is this workgroup's
    int seq = -1, q0 = 0, qlen = 0, qbase = 0;
    {
        int tile = blockIdx.x;
        for (int b = 0; b < a.batch; ++b) {
            const int lo = a.cu_seqlens_q ? a.cu_seqlens_q[b] : b, hi = a.cu_seqlens_q ? a.cu_seqlens_q[b + 1] : b + 1;
            const int tiles = (hi - lo + AQ - 1) / AQ;
            if (tile < tiles) {
                seq = b;
                q0 = tile * AQ;
                qlen = hi - lo;
                qbase = lo;
                break;
            }
            tile -= tiles;
        }
    }
    if (seq < 0) return;                                     // (uniform over the workgroup)
    const int head = blockIdx.y, kvh = head / (a.H / a.G);
    const int dim = a.dim, vdim = a.vdim;
    const int klen = a.context_lens[seq];
    const int past = klen - qlen;                            // keys before this step's first query
    const int nq = min(AQ, qlen - q0);
    const int kd = dim + 1, vd = vdim + 1;
    float* qs = smem;                                        // [AQ][dim]
    float* ks = qs + AQ * dim;                               // [AK][dim + 1]
    float* vs = ks + AK * kd;                                // [AK][vdim + 1]
    float* ps = vs + AK * vd;                                // [AQ][AK]
    const int tid = threadIdx.x, qi = tid >> 4, sub = tid & 15;
    for (int i = tid; i < AQ * dim; i += 256) {
        const int r = i / dim, d = i - r * dim;
        qs[i] = r < nq ? ldf((const A*)a.q, (int64_t)(qbase + q0 + r) * a.H * dim + head * dim + d) * a.scale : 0.f;
    }
    float acc[AVC];
#pragma unroll
    for (int c = 0; c < AVC; ++c) acc[c] = 0.f;
    // (a sink is what the row starts from: it has been seen with score sink, weight 1 and no value)
    float m_run = a.sinks ? a.sinks[head] : -INFINITY, l_run = a.sinks ? 1.f : 0.f;
    const int qpos = past + q0 + qi;                         // this lane's query position (valid for qi < nq)
    const int last_key = past + q0 + nq - 1;                 // the tile's last query sees keys 0..last_key
    const int32_t* table = a.block_tables + (int64_t)seq * a.table_stride;
    const float slope = a.slopes ? a.slopes[head] : 0.f;
    const TileWalk walk(a.window, a.keep_first, a.chunk, past + q0, AK);
    for (int k0 = walk.first_end > 0 || walk.win_start == 0 ? 0 : walk.win_start; k0 <= last_key; k0 = walk.next(k0)) {
        __syncthreads();                                     // the previous tile's readers are done
        for (int i = tid; i < AK * dim; i += 256) {
            const int r = i / dim, d = i - r * dim, key = k0 + r;
            float v = 0.f;
            if (key <= last_key) {
                const int64_t slot = (int64_t)table[key / a.page] * a.page + key % a.page;
                v = ldf((const A*)a.k_cache, (slot * a.G + kvh) * dim + d);
            }
            ks[r * kd + d] = v;
        }
        for (int i = tid; i < AK * vdim; i += 256) {
            const int r = i / vdim, d = i - r * vdim, key = k0 + r;
            float v = 0.f;
            if (key <= last_key) {
                v = ldf((const A*)a.v_cache, (((int64_t)table[key / a.page] * a.G + kvh) * vdim + d) * a.page + key % a.page);
            }
            vs[r * vd + d] = v;
        }
        __syncthreads();
        // scores of query qi against keys sub and sub + 16 of the tile
        float s0 = 0.f, s1 = 0.f;
        const float* qrow = qs + qi * dim;
        const float *kr0 = ks + sub * kd, *kr1 = ks + (sub + 16) * kd;
        for (int d = 0; d < dim; ++d) {
            const float qv = qrow[d];
            s0 = __builtin_fmaf(qv, kr0[d], s0);
            s1 = __builtin_fmaf(qv, kr1[d], s1);
        }
        const bool ok0 = qi < nq && key_visible(k0 + sub, qpos, a.window, a.keep_first, a.chunk), ok1 = qi < nq && key_visible(k0 + sub + 16, qpos, a.window, a.keep_first, a.chunk);
        s0 = ok0 ? s0 - slope * (float)(qpos - (k0 + sub)) : -INFINITY;
        s1 = ok1 ? s1 - slope * (float)(qpos - (k0 + sub + 16)) : -INFINITY;
        const float m_new = fmaxf(m_run, row16_max(fmaxf(s0, s1)));
        // a row that sees nothing yet keeps m = -inf (only rows past nq: every real query sees key 0)
        const float p0 = ok0 ? expf(s0 - m_new) : 0.f, p1 = ok1 ? expf(s1 - m_new) : 0.f;
        const float alpha = m_new == -INFINITY ? 1.f : expf(m_run - m_new);
        l_run = l_run * alpha + row16_sum(p0 + p1);
        m_run = m_new;
        ps[qi * AK + sub] = p0;
        ps[qi * AK + sub + 16] = p1;
        __syncthreads();
        const float* prow = ps + qi * AK;
#pragma unroll
        for (int c = 0; c < AVC; ++c) {
            const int col = sub + 16 * c;
            if (col < vdim) {
                float s = acc[c] * alpha;
                for (int r = 0; r < AK; ++r) s = __builtin_fmaf(prow[r], vs[r * vd + col], s);
                acc[c] = s;
            }
        }
    }
    // epilogue: normalise, turn back by the query's position, gate
    __syncthreads();
    float* os = ks;                                          // [AQ][vdim] (fits: AK >= AQ)
#pragma unroll
    for (int c = 0; c < AVC; ++c) {
        const int col = sub + 16 * c;
        if (col < vdim) os[qi * vdim + col] = l_run > 0.f ? acc[c] / l_run : 0.f;
    }
    __syncthreads();
    if (qi < nq) {
        const int64_t tok = qbase + q0 + qi;
        const float g = a.gate ? a.gate[tok * a.H + head] : 1.0f;
        const float pos = (float)qpos;
#pragma unroll
        for (int c = 0; c < AVC; ++c) {
            const int col = sub + 16 * c;
            if (col < vdim) {
                float v = os[qi * vdim + col];
                if (a.v_freq) {
                    int partner, pair;
                    bool first;
                    pair_of(col, vdim, a.v_interleaved, partner, pair, first);
                    const float o = os[qi * vdim + partner];
                    float sn, cs;
                    rot_sincos<A>(pos * a.v_freq[pair], sn, cs);
                    v = first ? v * cs + o * sn : v * cs - o * sn;        // the rotation by -pos
                }
                ((A*)a.out)[(tok * a.H + head) * vdim + col] = (A)(v * g);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// The same attention on the matrix cores, for bf16 caches with dim and vdim multiples of 16.  A workgroup is 64
// consecutive queries of one (sequence, head): four waves of 16 queries, all walking the same 64-key tiles (K rows and
// V transposed in LDS).  Per tile a wave forms S^T = K Q^T (lane: query lane%16, keys 4 (lane/16) + r of each 16-key
// block), keeps max / sum / weights in fp32, and accumulates O^T = V^T P^T with the weights as the B operand - as two
// bf16 terms, p = hi + lo, so a weight enters the product with 16 bits of mantissa and the sums stay fp32.  Tiles start
// at key 0 and every query has its own running maximum, so the result of a query does not depend on the cut or the batch.
typedef short s16x4 __attribute__((ext_vector_type(4)));
constexpr int MQ = 64, MK = 64;

// EXACT: dim == 16 NKS and vdim == 16 NVT, so no loop below carries a run-time bound (a guarded loop body is a branch, and the
// scheduler then cannot issue the LDS reads of several matrix instructions ahead of them).
// GROUPED (steps in which every sequence brings one query): a workgroup is one (sequence, KV head) and the 16 rows of a
// wave are the query heads that share this KV head, so its keys and values are read once for all of them; the four
// waves split every tile's keys and their partial results are merged at the end (the sums of a row are then formed in
// another order than in the other form: equal within fp32 rounding, not bit for bit).
// (The same split with 16 consecutive queries of one head as the rows was measured for prompts: no faster for one
// 1024-token chunk, 1.7-1.9 x slower from two chunks on, because it stages K/V four times as often.  Not kept.)
template <int NKS, int NVT, bool EXACT, int MODE>
__global__ __launch_bounds__(256) void attn_paged_mfma_kernel(AttnArgs a) {
    constexpr bool GROUPED = MODE == 1;                      // rows are the heads of a KV group (one query per sequence)
    constexpr bool SPLIT = MODE != 0;                        // the waves share 16 rows and split the keys
    constexpr int ROWS_Q = MQ;                               // queries per workgroup
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    int seq = -1, q0 = 0, qlen = 0, qbase = 0;
    {
        int tile = blockIdx.x;
        for (int b = 0; b < a.batch; ++b) {
            const int lo = a.cu_seqlens_q ? a.cu_seqlens_q[b] : b, hi = a.cu_seqlens_q ? a.cu_seqlens_q[b + 1] : b + 1;
            const int tiles = (hi - lo + ROWS_Q - 1) / ROWS_Q;
            if (tile < tiles) {
                seq = b;
                q0 = tile * ROWS_Q;
                qlen = hi - lo;
                qbase = lo;
                break;
            }
            tile -= tiles;
        }
    }
    if (seq < 0) return;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, fr = lane & 15, fq = lane >> 4;
    // GROUPED: blockIdx.y counts (KV head, part of its group of heads); the parts of one KV head read the same keys and values
    const int group = GROUPED ? a.H / (a.G * a.kv_split) : a.H / a.G;
    const int kvh = GROUPED ? blockIdx.y / a.kv_split : blockIdx.y / group;
    const int head = GROUPED ? blockIdx.y * group + min(fr, group - 1) : blockIdx.y;       // (GROUPED: this lane's row is a head)
    const int dim = a.dim, vdim = a.vdim, nks = dim >> 4, nvt = vdim >> 4;
    const int klen = a.context_lens[seq], past = klen - qlen;
    const int nq = GROUPED ? 1 : min(ROWS_Q, qlen - q0);
    const int nrows = GROUPED ? group : nq;                  // real rows of the workgroup's 64
    const int kld = dim + 8, vld = MK + 8;                   // LDS row strides in elements (8-byte aligned rows)
    bf16* ks = reinterpret_cast<bf16*>(smem_raw);            // [MK][dim + 8]
    bf16* vt = ks + MK * kld;                                // [vdim][MK + 8]: V transposed
    // GROUPED: every wave holds the same 16 rows (heads) and takes the 16 keys kt = wave of every 64-key tile, with its own
    // running maximum, sum and output; the four partial results are merged at the end.
    const int qrow = SPLIT ? fr : wave * 16 + fr;            // this lane's row within the workgroup
    const bool qok = qrow < nrows;
    constexpr int NKT = SPLIT ? 1 : 4;                       // 16-key blocks of a tile per wave
    const int qpos = GROUPED ? past : past + q0 + qrow;
    const int last_key = past + q0 + nq - 1;
    const int part = GROUPED ? (int)blockIdx.z : 0, nparts = GROUPED ? a.key_parts : 1;
    float* prow = nullptr;                                   // this workgroup's record among the parts
    if (GROUPED && nparts > 1) prow = a.parts + (((int64_t)seq * gridDim.y + blockIdx.y) * nparts + part) * 16 * (vdim + 2);
    if (last_key < 0 && prow) {                              // a padded row: every part records "no keys", the merge then writes zeros
        if (tid < 16) {
            prow[tid * (vdim + 2) + vdim] = -INFINITY;
            prow[tid * (vdim + 2) + vdim + 1] = 0.f;
        }
        return;
    }
    if (last_key < 0) {                                      // a padded row of a captured step (no keys): zeros, and no address is formed
        for (int i = tid; i < nrows * vdim; i += 256) {
            const int r = i / vdim;
            const int64_t tok = GROUPED ? qbase : qbase + q0 + r;
            const int hd = GROUPED ? (int)blockIdx.y * group + r : (int)blockIdx.y;
            ((bf16*)a.out)[(tok * a.H + hd) * vdim + (i - r * vdim)] = (bf16)0.f;
        }
        return;
    }
    const bf16* qg = (const bf16*)a.q + ((int64_t)(qbase + q0 + (qok && !GROUPED ? qrow : 0)) * a.H + head) * dim;
    s16x4 qf[NKS];
#pragma unroll
    for (int i = 0; i < NKS; ++i)
        if (EXACT || i < nks) qf[i] = *reinterpret_cast<const s16x4*>(qg + i * 16 + fq * 4);
    f32x4 o[NVT];
#pragma unroll
    for (int i = 0; i < NVT; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    if (a.sinks && (!SPLIT || (wave == 0 && part == 0))) {   // the sink is what a row starts from; where waves or parts share a row, one of them holds it
        m_run = a.sinks[head];
        l_run = 1.f;
    }
    const int32_t* table = a.block_tables + (int64_t)seq * a.table_stride;
    const bool wave_idle = !SPLIT && wave * 16 >= nrows;     // no row of this wave is real
    const int wave_last = SPLIT ? last_key : past + q0 + min(wave * 16 + 15, nq - 1);   // keys beyond it are masked for the whole wave
    // A tile's global loads (16 bytes each; K rows as they lie, V rows = value columns over 64 consecutive keys of one page)
    // are issued two tiles ahead into registers; addresses are clamped, what lies beyond the last key is zeroed on the way
    // into LDS.
    constexpr int KCH = (NKS + 1) / 2, VCH = (NVT + 1) / 2;  // 16-byte pieces per lane: MK * dim / 8 / 256
    const int kcols = dim >> 3;
    // The sequence's page ids go to LDS once: a tile's addresses then hang on no other load.  A tile lies within one page
    // (page % MK == 0).
    int* pages_s = reinterpret_cast<int*>(smem_raw + a.pages_offset);
    for (int i = tid; i <= last_key / a.page; i += 256) pages_s[i] = table[i];
    __syncthreads();
    auto fetch = [&](int k0, bf16x8 (&kpre)[KCH], bf16x8 (&vpre)[VCH]) {
        const int64_t pg = pages_s[k0 / a.page];
        const int in_page = k0 % a.page, rows = last_key - k0;       // (uniform)
#pragma unroll
        for (int j = 0; j < KCH; ++j) {
            const int i = tid + 256 * j;
            const int r = min(min(i / kcols, MK - 1), rows), c = (i % kcols) << 3;
            kpre[j] = *reinterpret_cast<const bf16x8*>((const bf16*)a.k_cache + (((pg * a.page + in_page + r) * a.G + kvh) * dim + c));
        }
        const int64_t vbase = (pg * a.G + kvh) * vdim;
#pragma unroll
        for (int j = 0; j < VCH; ++j) {
            const int i = tid + 256 * j;
            const int c = min(i >> 3, vdim - 1), piece = (i & 7) << 3;
            vpre[j] = *reinterpret_cast<const bf16x8*>((const bf16*)a.v_cache + (vbase + c) * a.page + k0 % a.page + piece);
        }
    };
    // Two register sets, two tiles ahead: the loads of the tile after next are issued when a tile has been handed to LDS.
    const float slope = a.slopes ? a.slopes[head] : 0.f;
    const TileWalk walk(a.window, a.keep_first, a.chunk, GROUPED ? past : past + q0, MK);
    bf16x8 kA[KCH], vA[VCH], kB[KCH], vB[VCH];
    // (with key parts a workgroup walks the tiles whose number is its own modulo the number of parts)
    auto mine = [&](int k0) { return nparts == 1 || (k0 / MK) % nparts == part; };
    auto next_tile = [&](int k0) {
        int n = walk.next(k0);
        while (n <= last_key && !mine(n)) n = walk.next(n);
        return n;
    };
    int ka = walk.first_end > 0 || walk.win_start == 0 ? 0 : walk.win_start;
    if (!mine(ka)) ka = next_tile(ka);
    int kb = next_tile(ka);
    if (ka > last_key) kb = ka;
    if (ka <= last_key) fetch(ka, kA, vA);
    if (kb <= last_key) fetch(kb, kB, vB);
    auto tile = [&](int k0, int k_after, bf16x8 (&kpre)[KCH], bf16x8 (&vpre)[VCH]) {
        __syncthreads();
#pragma unroll
        for (int j = 0; j < KCH; ++j) {
            const int i = tid + 256 * j;
            if (i < MK * kcols) {
                const int r = i / kcols, c = (i % kcols) << 3;
                *reinterpret_cast<bf16x8*>(ks + r * kld + c) = k0 + r <= last_key ? kpre[j] : bf16x8{};
            }
        }
#pragma unroll
        for (int j = 0; j < VCH; ++j) {
            const int i = tid + 256 * j;
            if (i < vdim * 8) {
                const int c = i >> 3, piece = (i & 7) << 3;
                bf16x8 v = vpre[j];
                if (k0 + MK - 1 > last_key) {                // (uniform: only the sequence's last tile)
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (k0 + piece + e > last_key) v[e] = (bf16)0.f;
                }
                *reinterpret_cast<bf16x8*>(vt + c * vld + piece) = v;
            }
        }
        __syncthreads();
        if (k_after <= last_key) fetch(k_after, kpre, vpre);
        if (wave_idle || k0 > wave_last) return;             // (wave-uniform; the barriers above are passed by all)
        f32x4 sc[NKT];
#pragma unroll
        for (int t = 0; t < NKT; ++t) {
            const int kt = SPLIT ? wave : t;
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < NKS; ++i)
                if (EXACT || i < nks) {
                    const s16x4 kf = *reinterpret_cast<const s16x4*>(ks + (kt * 16 + fr) * kld + i * 16 + fq * 4);
                    acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kf, qf[i], acc, 0, 0, 0);
                }
            sc[t] = acc;
        }
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = k0 + (SPLIT ? wave : t) * 16 + fq * 4 + r;
                const bool ok = qok && key_visible(key, qpos, a.window, a.keep_first, a.chunk);
                sc[t][r] = ok ? sc[t][r] * a.scale - slope * (float)(qpos - key) : -INFINITY;
                mx = fmaxf(mx, sc[t][r]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        // e^x as the hardware's 2^(x log2 e): fp32 throughout, about 1 ulp
        const float alpha = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f((m_run - m_new) * 1.4426950408889634f);
        float sum = 0.f;
        s16x4 ph[NKT], pl[NKT];
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float pv = sc[t][r] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((sc[t][r] - m_new) * 1.4426950408889634f);
                sum += pv;
                const bf16 hi = (bf16)pv;
                const bf16 lo = (bf16)(pv - (float)hi);
                ph[t][r] = __builtin_bit_cast(short, hi);
                pl[t][r] = __builtin_bit_cast(short, lo);
            }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        l_run = l_run * alpha + sum;
        m_run = m_new;
#pragma unroll
        for (int i = 0; i < NVT; ++i)
            if (EXACT || i < nvt) {
                f32x4 acc = o[i] * alpha;
#pragma unroll
                for (int t = 0; t < NKT; ++t) {
                    const int kt = SPLIT ? wave : t;
                    const s16x4 vf = *reinterpret_cast<const s16x4*>(vt + (i * 16 + fr) * vld + kt * 16 + fq * 4);
                    acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, ph[t], acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, pl[t], acc, 0, 0, 0);
                }
                o[i] = acc;
            }
    };
    while (ka <= last_key) {
        const int ka2 = next_tile(kb);
        tile(ka, ka2, kA, vA);
        if (kb > last_key) break;
        const int kb2 = next_tile(ka2);
        tile(kb, kb2, kB, vB);
        ka = ka2;
        kb = kb2;
    }
    // epilogue through LDS: [MQ][vdim] fp32, then turn back by the query's position, gate, store
    __syncthreads();
    float* os = reinterpret_cast<float*>(smem_raw);
    if constexpr (SPLIT) {
        // the four waves' partial results [wave][16 rows][vdim] and their (max, sum), merged into the first wave's rows
        float* ml = reinterpret_cast<float*>(smem_raw + a.ml_offset);
#pragma unroll
        for (int i = 0; i < NVT; ++i)
            if (EXACT || i < nvt)
#pragma unroll
                for (int r = 0; r < 4; ++r) os[(wave * 16 + fr) * vdim + i * 16 + fq * 4 + r] = o[i][r];
        if (fq == 0) {
            ml[(wave * 16 + fr) * 2] = m_run;
            ml[(wave * 16 + fr) * 2 + 1] = l_run;
        }
        __syncthreads();
        for (int i = tid; i < nrows * vdim; i += 256) {
            const int r = i / vdim, col = i - r * vdim;
            float big = -INFINITY;
#pragma unroll
            for (int w = 0; w < 4; ++w) big = fmaxf(big, ml[(w * 16 + r) * 2]);
            float num = 0.f, den = 0.f;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float mw = ml[(w * 16 + r) * 2];
                const float f = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((mw - big) * 1.4426950408889634f);
                num += os[(w * 16 + r) * vdim + col] * f;
                den += ml[(w * 16 + r) * 2 + 1] * f;
            }
            if (prow) {                                      // a part's record: the row relative to its maximum, then maximum and sum
                prow[r * (vdim + 2) + col] = num;
                if (col == 0) {
                    prow[r * (vdim + 2) + vdim] = big;
                    prow[r * (vdim + 2) + vdim + 1] = den;
                }
            } else {
                os[i] = den > 0.f ? num / den : 0.f;         // (element i of the first wave's rows: read above by this lane only)
            }
        }
        if (prow) return;                                    // (uniform) the merge launch finishes the rows
    } else {
        const float inv_l = l_run > 0.f ? 1.0f / l_run : 0.f;
#pragma unroll
        for (int i = 0; i < NVT; ++i)
            if (EXACT || i < nvt)
#pragma unroll
                for (int r = 0; r < 4; ++r) os[qrow * vdim + i * 16 + fq * 4 + r] = o[i][r] * inv_l;
    }
    __syncthreads();
    // one lane per rotation pair: both elements, one sine and cosine
    const int half = vdim >> 1;
    for (int i = tid; i < nrows * half; i += 256) {
        const int r = i / half, pair = i - r * half;
        const int c1 = a.v_interleaved ? 2 * pair : pair, c2 = a.v_interleaved ? 2 * pair + 1 : pair + half;
        const int64_t tok = GROUPED ? qbase : qbase + q0 + r;
        const int hd = GROUPED ? (int)blockIdx.y * group + r : (int)blockIdx.y;
        float u = os[r * vdim + c1], v = os[r * vdim + c2];
        if (a.v_freq) {
            float sn, cs;
            sincos_turns((float)(GROUPED ? past : past + q0 + r) * a.v_freq[pair], sn, cs);
            const float u2 = u * cs + v * sn;                // the rotation by -position
            v = v * cs - u * sn;
            u = u2;
        }
        const float g = a.gate ? a.gate[tok * a.H + hd] : 1.0f;
        bf16* dst = (bf16*)a.out + (tok * a.H + hd) * vdim;
        dst[c1] = (bf16)(u * g);
        dst[c2] = (bf16)(v * g);
    }
}

// The rows of the key parts of a (sequence, group of heads) merged: out = gate * sum_p num_p 2^(m_p - m) / sum_p den_p 2^(m_p - m).
__global__ __launch_bounds__(256) void attn_merge_parts_kernel(const float* __restrict__ parts, int nparts, int rows, int vdim, int H, const float* __restrict__ gate,
                                                               bf16* __restrict__ out) {
    // one workgroup per (sequence, group of heads, row): a lane per value column
    const int seq = blockIdx.x, hg = blockIdx.y, r = blockIdx.z;
    const float* base = parts + (((int64_t)seq * gridDim.y + hg) * nparts * 16 + r) * (vdim + 2);
    const int64_t pstride = (int64_t)16 * (vdim + 2);
    float big = -INFINITY;
    for (int p = 0; p < nparts; ++p) big = fmaxf(big, base[p * pstride + vdim]);
    const int hd = hg * rows + r;
    const float g = gate ? gate[(int64_t)seq * H + hd] : 1.0f;
    for (int col = threadIdx.x; col < vdim; col += 256) {
        float num = 0.f, den = 0.f;
        for (int p = 0; p < nparts; ++p) {
            const float* pr = base + p * pstride;
            if (pr[vdim] == -INFINITY) continue;             // a part without keys (its row is not written)
            const float f = __builtin_amdgcn_exp2f((pr[vdim] - big) * 1.4426950408889634f);
            num += pr[col] * f;
            den += pr[vdim + 1] * f;
        }
        out[((int64_t)seq * H + hd) * vdim + col] = (bf16)(den > 0.f ? num / den * g : 0.f);
    }
}

// One query per sequence: the heads of a KV group share a workgroup - up to 16 of them; a larger group is cut into parts.  A launch
// that would leave most of the chip idle is widened: where nothing turns the values back (no v_freq) by giving a sequence's key
// tiles to several workgroups in turn, whose rows a second launch merges (the keys and values are still read once); otherwise by
// cutting the group of heads further (its parts then read the same keys and values at about the same time).  Which workgroup a
// head or a tile falls to enters the result within fp32 rounding only (the order of the merge).
struct OneQueryPlan {
    int split, key_parts;
};
static OneQueryPlan one_query_plan(int64_t batch, int H, int G, bool turned_back) {
    const int group = H / G;
    int split = 1;
    while (group / split > 16 && group % (2 * split) == 0) split *= 2;
    int parts = 1;
    if (!turned_back) {
        while (batch * G * split * parts * 2 <= 256 && parts < 16) parts *= 2;       // (two workgroups a CU measured slower: 53 against 37 us)
    } else {
        while (batch * G * split < 256 && group % (2 * split) == 0 && group / split > 2) split *= 2;
    }
    return OneQueryPlan{split, parts};
}
static size_t one_query_parts_bytes(int64_t batch, int H, int G, int vdim, bool turned_back) {
    const OneQueryPlan pl = one_query_plan(batch, H, G, turned_back);
    return pl.key_parts > 1 ? sizeof(float) * (size_t)batch * G * pl.split * pl.key_parts * 16 * (vdim + 2) : 0;
}

template <int NKS, int NVT, bool EXACT>
static void launch_attn_mfma(const AttnArgs& a, int64_t total_q, hipStream_t st) {
    const size_t tiles = sizeof(bf16) * ((size_t)MK * (a.dim + 8) + (size_t)a.vdim * (MK + 8));
    const size_t outs = sizeof(float) * (size_t)MQ * a.vdim;
    AttnArgs b = a;
    b.pages_offset = (int)(((tiles > outs ? tiles : outs) + 15) & ~(size_t)15);
    b.ml_offset = (int)((b.pages_offset + sizeof(int) * (size_t)a.table_stride + 15) & ~(size_t)15);
    const size_t lds = b.ml_offset + sizeof(float) * 4 * 16 * 2;
    const int group = a.H / a.G;
    OneQueryPlan pl = one_query_plan(a.batch, a.H, a.G, a.v_freq != nullptr);
    if (!a.parts) pl.key_parts = 1;
    if (total_q == a.batch && group / pl.split <= 16 && !nvh_switch_on(SW_EXP_A)) {
        b.kv_split = pl.split;
        b.key_parts = pl.key_parts;
        attn_paged_mfma_kernel<NKS, NVT, EXACT, 1><<<dim3((unsigned)a.batch, (unsigned)(a.G * pl.split), (unsigned)pl.key_parts), 256, lds, st>>>(b);
        if (pl.key_parts > 1)
            attn_merge_parts_kernel<<<dim3((unsigned)a.batch, (unsigned)(a.G * pl.split), (unsigned)(group / pl.split)), 256, 0, st>>>(a.parts, pl.key_parts, group / pl.split, a.vdim, a.H, a.gate,
                                                                                                        (bf16*)a.out);
    } else {
        const dim3 grid((unsigned)(total_q / MQ + a.batch), (unsigned)a.H);
        attn_paged_mfma_kernel<NKS, NVT, EXACT, 0><<<grid, 256, lds, st>>>(b);
    }
}

// Exact instantiations for the head sizes in use (dim/16, vdim/16); any other 16-aligned pair takes a bounded one.
#define NVH_ATTN_EXACT(X) X(1, 1) X(2, 2) X(3, 3) X(4, 4) X(5, 5) X(6, 6) X(8, 8) X(12, 12) X(16, 16) X(2, 4) X(4, 2) X(4, 8) X(8, 4) X(8, 16) X(16, 8) X(12, 8) X(16, 12)
static void dispatch_attn_mfma(const AttnArgs& a, int64_t total_q, hipStream_t st) {
    const int nks = a.dim / 16, nvt = a.vdim / 16;
#define NVH_ATTN_CASE(K, V)                              \
    if (nks == K && nvt == V) {                          \
        launch_attn_mfma<K, V, true>(a, total_q, st);    \
        return;                                          \
    }
    NVH_ATTN_EXACT(NVH_ATTN_CASE)
#undef NVH_ATTN_CASE
    if (nks <= 4 && nvt <= 4) launch_attn_mfma<4, 4, false>(a, total_q, st);
    else if (nks <= 8 && nvt <= 8) launch_attn_mfma<8, 8, false>(a, total_q, st);
    else launch_attn_mfma<16, 16, false>(a, total_q, st);
}

}  // namespace

extern "C" int32_t nvh_attn_rotary_prep(const void* proj, int64_t proj_row_stride, const void* q_norm_weight, const void* k_norm_weight,
                                        float eps, const int64_t* positions, const float* qk_freq, float qk_mag, int64_t rot_dims,
                                        int32_t qk_interleaved, const float* v_freq, int32_t v_interleaved, void* q_out, float* gate_out,
                                        void* k_cache, void* v_cache, const int32_t* slot_mapping, int64_t page, int64_t num_tokens,
                                        int64_t num_q_heads, int64_t num_kv_heads, int64_t dim, int64_t vdim, int32_t norm_per_head, int32_t act_f32,
                                        nvh_stream_t stream) {
    NVH_REQUIRE(proj && positions && q_out && !q_norm_weight == !k_norm_weight, NVH_EINVAL, "nvh_attn_rotary_prep: null pointer");
    NVH_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && dim > 0 && vdim > 0 && num_tokens >= 0 && page > 0, NVH_EINVAL, "nvh_attn_rotary_prep: bad sizes");
    NVH_REQUIRE(rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0 && (rot_dims == 0 || qk_freq), NVH_EINVAL,
                "nvh_attn_rotary_prep: rot_dims %ld does not fit dim %ld", (long)rot_dims, (long)dim);
    NVH_REQUIRE(!v_freq || vdim % 2 == 0, NVH_EINVAL, "nvh_attn_rotary_prep: rotated values need an even vdim");
    NVH_REQUIRE(proj_row_stride >= (num_q_heads + num_kv_heads) * dim + num_kv_heads * vdim + (gate_out ? num_q_heads : 0), NVH_EINVAL,
                "nvh_attn_rotary_prep: projection row too short");
    if (num_tokens == 0) return NVH_OK;
    PrepArgs a{proj, proj_row_stride, q_norm_weight, k_norm_weight, norm_per_head, eps, positions, qk_freq, qk_mag, (int)rot_dims, qk_interleaved,
               v_freq, v_interleaved, q_out, gate_out, k_cache, v_cache, slot_mapping, (int)num_q_heads, (int)num_kv_heads, (int)dim, (int)vdim, (int)page};
    hipStream_t st = (hipStream_t)stream;
    const size_t lds = norm_per_head ? sizeof(float) * (size_t)(num_q_heads + num_kv_heads) : 0;
    NVH_REQUIRE(lds <= 32 * 1024, NVH_ENOSYS, "nvh_attn_rotary_prep: %ld heads above the per-head norm's limit", (long)(num_q_heads + num_kv_heads));
    if (act_f32) attn_rotary_prep_kernel<float><<<dim3((unsigned)num_tokens), 256, lds, st>>>(a);
    else attn_rotary_prep_kernel<bf16><<<dim3((unsigned)num_tokens), 256, lds, st>>>(a);
    NVH_CHECK_LAUNCH("nvh_attn_rotary_prep");
    return NVH_OK;
}

extern "C" int32_t nvh_attn_paged_any(const void* q, const void* k_cache, const void* v_cache, const int32_t* cu_seqlens_q,
                                      const int32_t* context_lens, const int32_t* block_tables, int64_t table_stride, int64_t batch,
                                      int64_t total_q, int64_t page, int64_t num_q_heads, int64_t num_kv_heads, int64_t dim, int64_t vdim,
                                      float scale, const float* gate, const float* v_freq, int32_t v_interleaved, const float* slopes,
                                      int64_t window, int64_t keep_first, int64_t chunk, const float* sinks, void* out, float* parts_ws,
                                      int64_t parts_ws_bytes, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(window >= 0 && keep_first >= 0 && window < (1 << 30) && keep_first < (1 << 30), NVH_EINVAL, "nvh_attn_paged_any: bad window");
    NVH_REQUIRE(chunk >= 0 && chunk < (1 << 30), NVH_EINVAL, "nvh_attn_paged_any: bad chunk");
    NVH_REQUIRE(q && k_cache && v_cache && context_lens && block_tables && out, NVH_EINVAL, "nvh_attn_paged_any: null pointer");
    NVH_REQUIRE(batch >= 0 && total_q >= 0 && page > 0 && num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0 && dim > 0 && vdim > 0,
                NVH_EINVAL, "nvh_attn_paged_any: bad sizes");
    NVH_REQUIRE(vdim <= 16 * AVC_MAX, NVH_ENOSYS, "nvh_attn_paged_any: vdim %ld above %d", (long)vdim, 16 * AVC_MAX);
    NVH_REQUIRE(!v_freq || vdim % 2 == 0, NVH_EINVAL, "nvh_attn_paged_any: rotated values need an even vdim");
    const size_t lds = sizeof(float) * (size_t)(AQ * dim + AK * (dim + 1) + AK * (vdim + 1) + AQ * AK);
    NVH_REQUIRE(lds <= 160 * 1024, NVH_ENOSYS, "nvh_attn_paged_any: dim %ld + vdim %ld need %zu bytes of LDS", (long)dim, (long)vdim, lds);
    if (lds > 64 * 1024) {                                   // beyond the default limit of dynamic LDS: raise it for both forms (gfx950: 160 KB per workgroup)
        const hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_paged_any_kernel<float, 16>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        const hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_paged_any_kernel<bf16, 16>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        const hipError_t e3 = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_paged_any_kernel<float, 32>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        const hipError_t e4 = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_paged_any_kernel<bf16, 32>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        NVH_REQUIRE(e1 == hipSuccess && e2 == hipSuccess && e3 == hipSuccess && e4 == hipSuccess, NVH_ENOSYS, "nvh_attn_paged_any: %zu bytes of LDS refused", lds);
    }
    if (batch == 0 || total_q == 0) return NVH_OK;
    AttnArgs a{q, k_cache, v_cache, cu_seqlens_q, context_lens, block_tables, table_stride, (int)batch, (int)page, (int)num_q_heads,
               (int)num_kv_heads, (int)dim, (int)vdim, scale, gate, v_freq, v_interleaved, out, slopes, (int)window, (int)keep_first, (int)chunk, sinks, 0, 0, 1, 1, nullptr};
    // at most ceil(len / AQ) tiles per sequence: total_q / AQ + batch bounds their number (surplus workgroups exit)
    const dim3 grid((unsigned)(total_q / AQ + batch), (unsigned)num_q_heads);
    hipStream_t st = (hipStream_t)stream;
    // bf16 with 16-aligned head sizes: the matrix-core kernel (the choice depends on the sizes and the type only)
    const bool mfma = !act_f32 && dim % 16 == 0 && vdim % 16 == 0 && dim <= 256 && vdim <= 256 && page % MK == 0 && nvh_aligned16(q) && nvh_aligned16(k_cache) &&
                      nvh_aligned16(v_cache) && !nvh_switch_on(SW_ATTN_ANY_NO_MFMA);
    if (mfma) {
        // (scratch for the key parts of the one-query form: used when it is given and large enough, see nvh_attn_paged_any_parts_bytes)
        const size_t need = total_q == batch ? one_query_parts_bytes(batch, (int)num_q_heads, (int)num_kv_heads, (int)vdim, v_freq != nullptr) : 0;
        if (parts_ws && need && (size_t)parts_ws_bytes >= need) a.parts = parts_ws;
        dispatch_attn_mfma(a, total_q, st);
    } else if (vdim <= 256) {                                // (16 value columns a lane; the choice depends on the size alone)
        if (act_f32) attn_paged_any_kernel<float, 16><<<grid, 256, lds, st>>>(a);
        else attn_paged_any_kernel<bf16, 16><<<grid, 256, lds, st>>>(a);
    } else {
        if (act_f32) attn_paged_any_kernel<float, 32><<<grid, 256, lds, st>>>(a);
        else attn_paged_any_kernel<bf16, 32><<<grid, 256, lds, st>>>(a);
    }
    NVH_CHECK_LAUNCH("nvh_attn_paged_any");
    return NVH_OK;
}

extern "C" int64_t nvh_attn_paged_any_parts_bytes(int64_t batch, int64_t total_q, int64_t num_q_heads, int64_t num_kv_heads, int64_t dim, int64_t vdim,
                                                  int64_t page, int32_t turned_back, int32_t act_f32) {
    if (batch <= 0 || total_q != batch || act_f32 || num_kv_heads <= 0 || num_q_heads % num_kv_heads) return 0;
    if (dim % 16 || vdim % 16 || dim > 256 || vdim > 256 || page % MK) return 0;           // (the matrix-core kernel's sizes)
    return (int64_t)one_query_parts_bytes(batch, (int)num_q_heads, (int)num_kv_heads, (int)vdim, turned_back != 0);
}
