// Mixture of experts: a token goes to the `top` experts whose router logits are largest, mixed with the weights that a
// softmax over just these `top` logits gives.
//   nvh_moe_route     fp32 router logits [T, E] -> expert ids and weights [T, top] (ties go to the lower expert id);
//                     nvh_moe_route_linear forms the logits itself (x W^T + b in fp32) in the same launch
//   nvh_moe_align     the (token, choice) pairs ordered by expert: for every position in that order the token it comes
//                     from, for every pair its position, and a list of 64-row tiles (expert, first position, rows) that
//                     covers every expert's block - all on the device, so a step never waits for the host and the whole
//                     layer can sit in a captured graph (the tile list has a fixed upper bound: pairs / 64 + experts)
//   nvh_gemm_grouped_any_nt   y[pos] = x[src(pos)] W[expert of pos]^T over that tile list: the any-shape product
//                     (gemm_any.h) with a weight matrix per tile and rows gathered through an index, bf16 on the matrix
//                     cores or true fp32.  A row's result does not depend on where in its expert's block it lies.
//   nvh_moe_combine   out fp32 [T, dim] = sum over a token's choices, in choice order, of weight * y[pos] (+ shared[t])
#include "common.h"
#include "gemm_any.h"

namespace {

// One wave per token: lane l holds logits l, l + 64, ...; `top` rounds of a wave-wide argmax.
constexpr int ROUTE_MAX_PER_LANE = 16;      // experts <= 1024

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int64_t stride, int32_t* __restrict__ ids, float* __restrict__ weights,
                                                        int64_t tokens, int experts, int top) {
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= tokens) return;
    const int lane = threadIdx.x & 63;
    float z[ROUTE_MAX_PER_LANE];
#pragma unroll
    for (int j = 0; j < ROUTE_MAX_PER_LANE; ++j) {
        const int e = lane + 64 * j;
        z[j] = e < experts ? logits[t * stride + e] : -INFINITY;
    }
    float first = 0.f, denom = 0.f;
    for (int r = 0; r < top; ++r) {
        float bv = -INFINITY;
        int be = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < ROUTE_MAX_PER_LANE; ++j) {
            const int e = lane + 64 * j;
            if (z[j] > bv || (z[j] == bv && e < be && z[j] != -INFINITY)) {
                bv = z[j];
                be = e;
            }
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int oe = __shfl_xor(be, off, 64);
            if (ov > bv || (ov == bv && oe < be)) {
                bv = ov;
                be = oe;
            }
        }
        if (r == 0) first = bv;
        const float w = expf(bv - first);                    // the first choice is the largest: exponents <= 0
        denom += w;
        if (lane == 0) {
            ids[t * top + r] = be;
            weights[t * top + r] = w;
        }
#pragma unroll
        for (int j = 0; j < ROUTE_MAX_PER_LANE; ++j)
            if (lane + 64 * j == be) z[j] = -INFINITY;       // taken
    }
    if (lane == 0)
        for (int r = 0; r < top; ++r) weights[t * top + r] = weights[t * top + r] / denom;
}

// The same with the router's product inside: z[e] = x . w[e] + bias[e] in fp32, every expert's dot product spread over the
// wave's lanes (lane l takes elements l, l + 64, ... of the row) and summed across it.
// One workgroup per token: its four waves take the experts four at a time in turn, every dot product spread over a wave's
// lanes (a lane takes 8 consecutive elements of every 512) and summed across it; the logits meet in LDS and the first wave picks.
template <typename A>
__global__ __launch_bounds__(256) void moe_route_linear_kernel(const A* __restrict__ x, int64_t ldx, const A* __restrict__ w, const A* __restrict__ bias,
                                                               int32_t* __restrict__ ids, float* __restrict__ weights, float* __restrict__ logits_out,
                                                               int experts, int K, int top, int vec, int sigmoid_scores) {
    __shared__ float zs[64 * ROUTE_MAX_PER_LANE];
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const A* xr = x + t * ldx;
    constexpr int EG = 4;
    for (int e0 = wave * EG; e0 < experts; e0 += 4 * EG) {
        float acc[EG];
#pragma unroll
        for (int g = 0; g < EG; ++g) acc[g] = 0.f;
        for (int k0 = lane * 8; k0 < K; k0 += 512) {
            float xv[8];
            nvh_load8(xr, k0, K - k0, vec, xv);
#pragma unroll
            for (int g = 0; g < EG; ++g) {
                float wv[8];
                nvh_load8(w + (int64_t)min(e0 + g, experts - 1) * K, k0, K - k0, vec, wv);
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[g] = __builtin_fmaf(xv[i], wv[i], acc[g]);
            }
        }
#pragma unroll
        for (int g = 0; g < EG; ++g) {
            const int e = e0 + g;
            const float s = wave_sum(acc[g]) + (bias && e < experts ? (float)bias[e] : 0.f);
            if (lane == 0 && e < experts) {
                zs[e] = s;
                if (logits_out) logits_out[t * experts + e] = s;
            }
        }
    }
    __syncthreads();
    if (wave != 0) return;
    float z[ROUTE_MAX_PER_LANE];
#pragma unroll
    for (int j = 0; j < ROUTE_MAX_PER_LANE; ++j) z[j] = lane + 64 * j < experts ? zs[lane + 64 * j] : -INFINITY;
    float first = 0.f, denom = 0.f;
    for (int r = 0; r < top; ++r) {
        float bv = -INFINITY;
        int be = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < ROUTE_MAX_PER_LANE; ++j) {
            const int e = lane + 64 * j;
            if (z[j] > bv || (z[j] == bv && e < be && z[j] != -INFINITY)) {
                bv = z[j];
                be = e;
            }
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int oe = __shfl_xor(be, off, 64);
            if (ov > bv || (ov == bv && oe < be)) {
                bv = ov;
                be = oe;
            }
        }
        if (r == 0) first = bv;
        // (sigmoid scores: an expert's weight is its own score, whatever the others'; the order by logit is the order by score)
        const float wgt = sigmoid_scores ? 1.0f / (1.0f + expf(-bv)) : expf(bv - first);
        denom += wgt;
        if (lane == 0) {
            ids[t * top + r] = be;
            weights[t * top + r] = wgt;
        }
#pragma unroll
        for (int j = 0; j < ROUTE_MAX_PER_LANE; ++j)
            if (lane + 64 * j == be) z[j] = -INFINITY;
    }
    if (lane == 0 && !sigmoid_scores)
        for (int r = 0; r < top; ++r) weights[t * top + r] = weights[t * top + r] / denom;
}

// Routing by scores: s = softmax(x W^T) over ALL experts; the choice goes by s + correction (a per-expert offset that
// does not enter the weights), optionally restricted to groups of neighbouring experts - a group's score is its largest
// choice score and only the `keep` best groups stay eligible (the others count as minus infinity); the `top` best eligible
// experts are taken (ties: lower id) and weighted by their s times `scale`, not renormalised.  `aux` [n_aux, K]: further
// rows that read the same input; their fp32 products go to aux_out [T, n_aux] (a gate of the layer, say).
// One workgroup per token, products as in moe_route_linear_kernel; the first wave picks.
// PL: experts (and groups) a lane of the picking wave holds: experts <= 64 PL.
template <typename A, int PL>
__global__ __launch_bounds__(256) void moe_route_scored_kernel(const A* __restrict__ x, int64_t ldx, const A* __restrict__ w, const A* __restrict__ correction,
                                                               const A* __restrict__ aux, float* __restrict__ aux_out, int n_aux, int32_t* __restrict__ ids,
                                                               float* __restrict__ weights, float* __restrict__ scores_out, int experts, int K, int top,
                                                               int groups, int keep, float scale, int vec) {
    __shared__ float zs[64 * PL];            // logits, then scores
    __shared__ float cs[64 * PL];            // choice scores
    __shared__ float gsc[64 * PL];           // 1 for a kept group
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const A* xr = x + t * ldx;
    // every wave takes `eg` rows at a time (up to EG: 17 rows are one pass of five a wave, not two passes of four)
    constexpr int EG = 8;
    const int rows = experts + n_aux;
    const int eg = min(EG, (rows + 3) / 4);
    for (int e0 = wave * eg; e0 < rows; e0 += 4 * eg) {
        float acc[EG];
#pragma unroll
        for (int g = 0; g < EG; ++g) acc[g] = 0.f;
        for (int k0 = lane * 8; k0 < K; k0 += 512) {
            float xv[8];
            nvh_load8(xr, k0, K - k0, vec, xv);
#pragma unroll
            for (int g = 0; g < EG; ++g)
                if (g < eg) {                                // (uniform)
                    const int e = min(e0 + g, rows - 1);
                    const A* wr = e < experts ? w + (int64_t)e * K : aux + (int64_t)(e - experts) * K;
                    float wv[8];
                    nvh_load8(wr, k0, K - k0, vec, wv);
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc[g] = __builtin_fmaf(xv[i], wv[i], acc[g]);
                }
        }
#pragma unroll
        for (int g = 0; g < EG; ++g)
            if (g < eg) {
                const int e = e0 + g;
                const float sum = wave_sum(acc[g]);
                if (lane == 0 && e < experts) zs[e] = sum;
                else if (lane == 0 && e < rows) aux_out[t * n_aux + (e - experts)] = sum;
            }
    }
    __syncthreads();
    const bool picker = wave == 0;                           // the first wave picks; the others only keep the barriers company
    // softmax over all experts
    float z[PL];
    if (picker) {
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < PL; ++j) {
            z[j] = lane + 64 * j < experts ? zs[lane + 64 * j] : -INFINITY;
            mx = fmaxf(mx, z[j]);
        }
        mx = wave_max(mx);
        float den = 0.f;
#pragma unroll
        for (int j = 0; j < PL; ++j) {
            z[j] = lane + 64 * j < experts ? expf(z[j] - mx) : 0.f;
            den += z[j];
        }
        den = wave_sum(den);
#pragma unroll
        for (int j = 0; j < PL; ++j) {
            const int e = lane + 64 * j;
            if (e < experts) {
                const float sc = z[j] / den;
                zs[e] = sc;
                if (scores_out) scores_out[t * experts + e] = sc;
                z[j] = sc + (correction ? (float)correction[e] : 0.f);
                cs[e] = z[j];
            } else {
                z[j] = -INFINITY;
            }
        }
    }
    __syncthreads();
    if (groups > 1 && keep < groups) {                       // (uniform)
        const int gsz = experts / groups;
        float gv[PL];
        bool gone[PL];
        if (picker) {
#pragma unroll
            for (int j = 0; j < PL; ++j) {
                const int g = lane + 64 * j;
                gone[j] = g >= groups;
                gv[j] = -INFINITY;
                if (g < groups) {
                    for (int i = 0; i < gsz; ++i) gv[j] = fmaxf(gv[j], cs[g * gsz + i]);
                    gsc[g] = 0.f;                            // becomes 1 for a kept group
                }
            }
        }
        __syncthreads();
        if (picker) {
            for (int r = 0; r < keep; ++r) {
                float bv = -INFINITY;
                int bg = 0x7fffffff;
#pragma unroll
                for (int j = 0; j < PL; ++j)
                    if (!gone[j] && (bg == 0x7fffffff || gv[j] > bv)) {
                        bv = gv[j];
                        bg = lane + 64 * j;
                    }
#pragma unroll
                for (int off = 1; off < 64; off <<= 1) {
                    const float ov = __shfl_xor(bv, off, 64);
                    const int og = __shfl_xor(bg, off, 64);
                    if (og != 0x7fffffff && (bg == 0x7fffffff || ov > bv || (ov == bv && og < bg))) {
                        bv = ov;
                        bg = og;
                    }
                }
                if (lane == 0) gsc[bg] = 1.f;
#pragma unroll
                for (int j = 0; j < PL; ++j)
                    if (lane + 64 * j == bg) gone[j] = true;
            }
        }
        __syncthreads();
        if (picker) {
#pragma unroll
            for (int j = 0; j < PL; ++j) {
                const int e = lane + 64 * j;
                if (e < experts && gsc[e / gsz] == 0.f) z[j] = -INFINITY;
            }
        }
    }
    if (!picker) return;
    bool taken[PL];
#pragma unroll
    for (int j = 0; j < PL; ++j) taken[j] = lane + 64 * j >= experts;
    for (int r = 0; r < top; ++r) {
        float bv = -INFINITY;
        int be = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < PL; ++j) {
            const int e = lane + 64 * j;
            if (!taken[j] && (z[j] > bv || be == 0x7fffffff)) {
                bv = z[j];
                be = e;
            }
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int oe = __shfl_xor(be, off, 64);
            if (oe != 0x7fffffff && (be == 0x7fffffff || ov > bv || (ov == bv && oe < be))) {
                bv = ov;
                be = oe;
            }
        }
        if (lane == 0) {
            ids[t * top + r] = be;
            weights[t * top + r] = zs[be] * scale;
        }
#pragma unroll
        for (int j = 0; j < PL; ++j)
            if (lane + 64 * j == be) taken[j] = true;
    }
}

// One workgroup: counts per expert, block starts, then every pair takes the next free position of its expert's block.
// (Which position a pair gets within its block depends on the order the lanes arrive in; nothing downstream depends on it.)
__global__ __launch_bounds__(1024) void moe_align_kernel(const int32_t* __restrict__ ids, int64_t pairs, int experts, int top, int32_t* __restrict__ src_token,
                                                         int32_t* __restrict__ pos_of_pair, int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row0,
                                                         int32_t* __restrict__ tile_rows, int max_tiles) {
    extern __shared__ int sh[];                              // [experts] counts, [experts] starts / cursors, [experts] first tile
    int* count = sh;
    int* start = sh + experts;
    int* tile0 = sh + 2 * experts;
    for (int e = threadIdx.x; e < experts; e += 1024) count[e] = 0;
    __syncthreads();
    for (int64_t i = threadIdx.x; i < pairs; i += 1024) {
        const int e = ids[i];
        if (e >= 0 && e < experts) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int row = 0, tile = 0;
        for (int e = 0; e < experts; ++e) {
            start[e] = row;
            tile0[e] = tile;
            row += count[e];
            tile += (count[e] + nvh_any::GT - 1) / nvh_any::GT;
        }
        tile0[experts] = tile;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < max_tiles; i += 1024) tile_rows[i] = 0;
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += 1024) {
        const int n = count[e];
        for (int k = 0, t = tile0[e]; k < n && t < max_tiles; k += nvh_any::GT, ++t) {
            tile_expert[t] = e;
            tile_row0[t] = start[e] + k;
            tile_rows[t] = min(nvh_any::GT, n - k);
        }
    }
    __syncthreads();
    for (int64_t i = threadIdx.x; i < pairs; i += 1024) {
        const int e = ids[i];
        if (e < 0 || e >= experts) {
            pos_of_pair[i] = -1;
            continue;
        }
        const int pos = atomicAdd(&start[e], 1);
        src_token[pos] = (int32_t)(i / top);
        pos_of_pair[i] = pos;
    }
}

struct GroupedArgs {
    const void* x;             // rows of K
    int64_t ldx;
    const int32_t* gather;     // [pairs]: source row of x for every output row (null: the output row's own index)
    const void* w;             // [experts, N, K]
    void* y;                   // [pairs, N]
    int64_t ldy;
    const int32_t *tile_expert, *tile_row0, *tile_rows;
    int N, K, vec_ok;
};

template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_grouped_bf16_kernel(GroupedArgs a) {
    const int rows = a.tile_rows[blockIdx.y];
    if (rows <= 0) return;                                   // (uniform: a tile beyond the list's end)
    const bf16* w = (const bf16*)a.w + (int64_t)a.tile_expert[blockIdx.y] * a.N * a.K;
    nvh_any::gemm_any_bf16_tile<OUT_F32>((const bf16*)a.x, a.ldx, w, a.K, nullptr, a.y, a.ldy, nvh_any::RowMap{a.gather, a.tile_row0[blockIdx.y], rows},
                                         blockIdx.x * nvh_any::GT, a.N, a.K, a.vec_ok);
}

__global__ __launch_bounds__(256) void gemm_grouped_f32_kernel(GroupedArgs a) {
    const int rows = a.tile_rows[blockIdx.y];
    if (rows <= 0) return;
    const float* w = (const float*)a.w + (int64_t)a.tile_expert[blockIdx.y] * a.N * a.K;
    nvh_any::gemm_any_f32_tile((const float*)a.x, a.ldx, w, a.K, nullptr, (float*)a.y, a.ldy, nvh_any::RowMap{a.gather, a.tile_row0[blockIdx.y], rows},
                               blockIdx.x * nvh_any::GT, a.N, a.K);
}

template <typename A>
__global__ __launch_bounds__(256) void moe_combine_kernel(const A* __restrict__ y, int64_t ldy, const int32_t* __restrict__ pos_of_pair, const float* __restrict__ weights,
                                                          const A* __restrict__ shared, int64_t shared_stride, const float* __restrict__ shared_gate,
                                                          int64_t gate_stride, float* __restrict__ out, int dim, int top) {
    const int64_t t = blockIdx.x;
    const float sg = shared_gate ? 1.0f / (1.0f + expf(-shared_gate[t * gate_stride])) : 1.0f;
    for (int c = threadIdx.x; c < dim; c += 256) {
        float s = 0.f;
        for (int r = 0; r < top; ++r) {
            const int pos = pos_of_pair[t * top + r];
            if (pos >= 0) s = __builtin_fmaf(weights ? weights[t * top + r] : 1.0f, (float)y[(int64_t)pos * ldy + c], s);
        }
        if (shared) s += sg * (float)shared[t * shared_stride + c];
        out[t * dim + c] = s;
    }
}

// The experts' activation where a pair's routing weight multiplies the expert's INPUT: the rows of the first grouped product were
// formed from the unweighted token, and since that product is linear, row * weight is the product of the weighted token.  Then, with
// the gate's value capped above and the other half's value clamped to +-limit,
//   g = min(w G, limit);  u = clamp(w U, -limit, limit);  y = g sigmoid(alpha g) (u + 1).
// One workgroup per (token, choice) pair; its row is pos_of_pair[pair] (< 0: the pair has no row).
template <typename A>
__global__ __launch_bounds__(256) void glu_clamp_pairs_kernel(const A* __restrict__ gu, int64_t gu_stride, const int32_t* __restrict__ pos_of_pair,
                                                              const float* __restrict__ weights, A* __restrict__ y, int64_t y_stride, int inter, float limit,
                                                              float alpha) {
    const int64_t pair = blockIdx.x;
    const int pos = pos_of_pair[pair];
    if (pos < 0) return;
    const float w = weights ? weights[pair] : 1.0f;
    const A* row = gu + (int64_t)pos * gu_stride;
    for (int c = threadIdx.x; c < inter; c += 256) {
        const float g = fminf((float)row[c] * w, limit);
        const float u = fminf(fmaxf((float)row[inter + c] * w, -limit), limit);
        y[(int64_t)pos * y_stride + c] = (A)(g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
    }
}

}  // namespace

extern "C" int32_t nvh_moe_route(const float* logits, int64_t row_stride, int32_t* ids, float* weights, int64_t num_tokens, int64_t experts,
                                 int64_t top, nvh_stream_t stream) {
    NVH_REQUIRE(logits && ids && weights, NVH_EINVAL, "nvh_moe_route: null pointer");
    NVH_REQUIRE(num_tokens >= 0 && experts > 0 && top > 0 && top <= experts && row_stride >= experts, NVH_EINVAL, "nvh_moe_route: bad sizes");
    NVH_REQUIRE(experts <= 64 * ROUTE_MAX_PER_LANE, NVH_ENOSYS, "nvh_moe_route: %ld experts above %d", (long)experts, 64 * ROUTE_MAX_PER_LANE);
    if (num_tokens == 0) return NVH_OK;
    moe_route_kernel<<<dim3((unsigned)nvh_cdiv(num_tokens, 4)), 256, 0, (hipStream_t)stream>>>(logits, row_stride, ids, weights, num_tokens, (int)experts, (int)top);
    NVH_CHECK_LAUNCH("nvh_moe_route");
    return NVH_OK;
}

extern "C" int32_t nvh_moe_route_linear(const void* x, int64_t x_row_stride, const void* w, const void* bias, int32_t* ids, float* weights,
                                        float* logits_out, int64_t num_tokens, int64_t experts, int64_t K, int64_t top, int32_t sigmoid_scores,
                                        int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(x && w && ids && weights, NVH_EINVAL, "nvh_moe_route_linear: null pointer");
    NVH_REQUIRE(num_tokens >= 0 && experts > 0 && top > 0 && top <= experts && K > 0 && K < (1 << 30) && x_row_stride >= K, NVH_EINVAL, "nvh_moe_route_linear: bad sizes");
    NVH_REQUIRE(experts <= 64 * ROUTE_MAX_PER_LANE, NVH_ENOSYS, "nvh_moe_route_linear: %ld experts above %d", (long)experts, 64 * ROUTE_MAX_PER_LANE);
    if (num_tokens == 0) return NVH_OK;
    const dim3 grid((unsigned)num_tokens);
    hipStream_t st = (hipStream_t)stream;
    const int vec = K % 8 == 0 && x_row_stride % 8 == 0 && nvh_aligned16(x) && nvh_aligned16(w);
    if (act_f32) moe_route_linear_kernel<float><<<grid, 256, 0, st>>>((const float*)x, x_row_stride, (const float*)w, (const float*)bias, ids, weights, logits_out, (int)experts, (int)K, (int)top, vec, sigmoid_scores);
    else moe_route_linear_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)x, x_row_stride, (const bf16*)w, (const bf16*)bias, ids, weights, logits_out, (int)experts, (int)K, (int)top, vec, sigmoid_scores);
    NVH_CHECK_LAUNCH("nvh_moe_route_linear");
    return NVH_OK;
}

extern "C" int32_t nvh_moe_route_scored(const void* x, int64_t x_row_stride, const void* w, const void* correction, const void* aux, float* aux_out,
                                        int64_t num_aux, int32_t* ids, float* weights, float* scores_out, int64_t num_tokens, int64_t experts, int64_t K,
                                        int64_t top, int64_t groups, int64_t keep, float scale, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(x && w && ids && weights && (num_aux == 0 || (aux && aux_out)), NVH_EINVAL, "nvh_moe_route_scored: null pointer");
    NVH_REQUIRE(num_tokens >= 0 && experts > 0 && top > 0 && top <= experts && K > 0 && K < (1 << 30) && x_row_stride >= K && num_aux >= 0 && num_aux <= 64, NVH_EINVAL,
                "nvh_moe_route_scored: bad sizes");
    NVH_REQUIRE(groups >= 1 && experts % groups == 0 && keep >= 1 && keep <= groups && top <= keep * (experts / groups), NVH_EINVAL,
                "nvh_moe_route_scored: %ld groups (keep %ld) do not fit %ld experts, top %ld", (long)groups, (long)keep, (long)experts, (long)top);
    NVH_REQUIRE(experts <= 64 * ROUTE_MAX_PER_LANE, NVH_ENOSYS, "nvh_moe_route_scored: %ld experts above %d", (long)experts, 64 * ROUTE_MAX_PER_LANE);
    if (num_tokens == 0) return NVH_OK;
    const dim3 grid((unsigned)num_tokens);
    hipStream_t st = (hipStream_t)stream;
    const int vec = K % 8 == 0 && x_row_stride % 8 == 0 && nvh_aligned16(x) && nvh_aligned16(w) && (!aux || nvh_aligned16(aux));
#define NVH_ROUTE_SCORED(A, PL) moe_route_scored_kernel<A, PL><<<grid, 256, 0, st>>>((const A*)x, x_row_stride, (const A*)w, (const A*)correction, (const A*)aux, aux_out, (int)num_aux, ids, weights, scores_out, (int)experts, (int)K, (int)top, (int)groups, (int)keep, scale, vec)
    if (experts <= 64) {
        if (act_f32) NVH_ROUTE_SCORED(float, 1);
        else NVH_ROUTE_SCORED(bf16, 1);
    } else if (experts <= 256) {
        if (act_f32) NVH_ROUTE_SCORED(float, 4);
        else NVH_ROUTE_SCORED(bf16, 4);
    } else {
        if (act_f32) NVH_ROUTE_SCORED(float, ROUTE_MAX_PER_LANE);
        else NVH_ROUTE_SCORED(bf16, ROUTE_MAX_PER_LANE);
    }
#undef NVH_ROUTE_SCORED
    NVH_CHECK_LAUNCH("nvh_moe_route_scored");
    return NVH_OK;
}

extern "C" int64_t nvh_moe_max_tiles(int64_t pairs, int64_t experts) { return pairs / nvh_any::GT + experts; }

extern "C" int32_t nvh_moe_align(const int32_t* ids, int64_t num_tokens, int64_t experts, int64_t top, int32_t* src_token, int32_t* pos_of_pair,
                                 int32_t* tile_expert, int32_t* tile_row0, int32_t* tile_rows, int64_t max_tiles, nvh_stream_t stream) {
    NVH_REQUIRE(ids && src_token && pos_of_pair && tile_expert && tile_row0 && tile_rows, NVH_EINVAL, "nvh_moe_align: null pointer");
    NVH_REQUIRE(num_tokens >= 0 && experts > 0 && experts <= 4096 && top > 0 && max_tiles >= nvh_moe_max_tiles(num_tokens * top, experts) && num_tokens * top < (1 << 30),
                NVH_EINVAL, "nvh_moe_align: bad sizes");
    if (num_tokens == 0) return NVH_OK;
    const size_t lds = sizeof(int) * (size_t)(3 * experts + 1);
    moe_align_kernel<<<dim3(1), 1024, lds, (hipStream_t)stream>>>(ids, num_tokens * top, (int)experts, (int)top, src_token, pos_of_pair, tile_expert, tile_row0,
                                                                  tile_rows, (int)max_tiles);
    NVH_CHECK_LAUNCH("nvh_moe_align");
    return NVH_OK;
}

extern "C" int32_t nvh_gemm_grouped_any_nt(const void* x, int64_t x_row_stride, const int32_t* gather, const void* w, void* y, int64_t y_row_stride,
                                           const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* tile_rows, int64_t max_tiles,
                                           int64_t N, int64_t K, int32_t in_f32, int32_t out_f32, nvh_stream_t stream) {
    NVH_REQUIRE(x && w && y && tile_expert && tile_row0 && tile_rows, NVH_EINVAL, "nvh_gemm_grouped_any_nt: null pointer");
    NVH_REQUIRE(max_tiles >= 0 && max_tiles < 65536 && N > 0 && K > 0 && N < (1 << 30) && K < (1 << 30) && x_row_stride >= K && y_row_stride >= N, NVH_EINVAL,
                "nvh_gemm_grouped_any_nt: bad sizes");
    NVH_REQUIRE(!in_f32 || out_f32, NVH_ENOSYS, "nvh_gemm_grouped_any_nt: fp32 operands give an fp32 product");
    if (max_tiles == 0) return NVH_OK;
    const int vec_ok = !in_f32 && K % 8 == 0 && x_row_stride % 8 == 0 && nvh_aligned16(x) && nvh_aligned16(w);
    const GroupedArgs a{x, x_row_stride, gather, w, y, y_row_stride, tile_expert, tile_row0, tile_rows, (int)N, (int)K, vec_ok};
    const dim3 grid((unsigned)nvh_cdiv(N, nvh_any::GT), (unsigned)max_tiles);
    hipStream_t st = (hipStream_t)stream;
    if (in_f32) gemm_grouped_f32_kernel<<<grid, 256, 0, st>>>(a);
    else if (out_f32) gemm_grouped_bf16_kernel<true><<<grid, 256, 0, st>>>(a);
    else gemm_grouped_bf16_kernel<false><<<grid, 256, 0, st>>>(a);
    NVH_CHECK_LAUNCH("nvh_gemm_grouped_any_nt");
    return NVH_OK;
}

extern "C" int32_t nvh_glu_clamp_pairs(const void* gate_up, int64_t row_stride, const int32_t* pos_of_pair, const float* weights, void* y, int64_t y_stride,
                                       int64_t pairs, int64_t inter, float limit, float alpha, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(gate_up && pos_of_pair && y && pairs >= 0 && inter > 0 && row_stride >= 2 * inter && y_stride >= inter && limit > 0.f, NVH_EINVAL,
                "nvh_glu_clamp_pairs: bad argument");
    if (pairs == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) glu_clamp_pairs_kernel<float><<<dim3((unsigned)pairs), 256, 0, st>>>((const float*)gate_up, row_stride, pos_of_pair, weights, (float*)y, y_stride, (int)inter, limit, alpha);
    else glu_clamp_pairs_kernel<bf16><<<dim3((unsigned)pairs), 256, 0, st>>>((const bf16*)gate_up, row_stride, pos_of_pair, weights, (bf16*)y, y_stride, (int)inter, limit, alpha);
    NVH_CHECK_LAUNCH("nvh_glu_clamp_pairs");
    return NVH_OK;
}

extern "C" int32_t nvh_moe_combine(const void* y, int64_t y_row_stride, const int32_t* pos_of_pair, const float* weights, const void* shared,
                                   int64_t shared_stride, const float* shared_gate, int64_t shared_gate_stride, float* out, int64_t num_tokens, int64_t dim,
                                   int64_t top, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(y && pos_of_pair && out && num_tokens >= 0 && dim > 0 && top > 0 && y_row_stride >= dim, NVH_EINVAL, "nvh_moe_combine: bad argument");
    if (num_tokens == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) moe_combine_kernel<float><<<dim3((unsigned)num_tokens), 256, 0, st>>>((const float*)y, y_row_stride, pos_of_pair, weights, (const float*)shared, shared_stride, shared_gate, shared_gate_stride, out, (int)dim, (int)top);
    else moe_combine_kernel<bf16><<<dim3((unsigned)num_tokens), 256, 0, st>>>((const bf16*)y, y_row_stride, pos_of_pair, weights, (const bf16*)shared, shared_stride, shared_gate, shared_gate_stride, out, (int)dim, (int)top);
    NVH_CHECK_LAUNCH("nvh_moe_combine");
    return NVH_OK;
}
