// Attention through a low-rank latent: what a token leaves in the cache is one normed latent vector c (kv_rank wide) and one
// rotated key part shared by all heads (rot wide); every head's unrotated key W_uk c and value W_uv c are linear in c, so
// neither is ever formed.  With q_h = [q_n | q_r] the score is
//     q_n . (W_uk,h c) + q_r . k_r  =  (W_uk,h^T q_n) . c + q_r . k_r,
// i.e. plain attention of the query [W_uk,h^T q_n | q_r] over the key [c | k_r] with ONE key/value head that all query
// heads share, whose value is c itself; a head's output is then W_uv,h applied to its weighted sum of latents.
//   nvh_latent_prep      per token, over the fused projection row [dq | dkv | gate]: RMS norm (with weight) of the query
//                        latent; RMS norm of the key/value latent and interleaved-or-half rotary of the shared key part,
//                        both written to the token's cache slot (keys [pages, page, 1, kv_rank + rot], values = the latent
//                        once more, transposed within a page as the paged attention wants them); sigmoid of the head gates
//   nvh_gemm_heads_nt    y[t, h, :] = x[t, h, :] W[h]^T for every head (the any-shape product's tile, gemm_any.h, with a
//                        weight matrix per head): the absorption of W_uk into the query and of W_uv into the output
//   nvh_latent_q_rotary  rotary of every head's rotated query part into its place behind the absorbed part
// The attention itself is nvh_attn_paged_any (attention_any.hip).
#include "common.h"
#include "gemm_any.h"

namespace {

__device__ __forceinline__ float block_sum_256(float v, float* scratch) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    return scratch[0] + scratch[1] + scratch[2] + scratch[3];
}

struct LatentPrepArgs {
    const void* proj;          // [T, ld]: dq (q_rank) | dkv (kv_rank + rot; absent without own_kv) | gate (H; absent without gate_out)
    int64_t ld;
    int q_rank, kv_rank, rot, H, own_kv;
    const void *q_norm, *kv_norm;   // [q_rank], [kv_rank]
    float eps;
    const int64_t* positions;
    const float* freq;         // [rot / 2]
    float mag;
    int interleaved;
    void* cq_out;              // [T, q_rank]
    float* gate_out;           // [T, H] or null
    void *k_cache, *v_cache;   // [pages, page, 1, kv_rank + rot], [pages, 1, kv_rank, page]
    const int32_t* slot_mapping;
    int page;
};

template <typename A>
__global__ __launch_bounds__(256) void latent_prep_kernel(LatentPrepArgs a) {
    __shared__ float red[4];
    const int64_t t = blockIdx.x;
    const A* row = (const A*)a.proj + t * a.ld;
    const A* dq = row;
    const A* dkv = row + a.q_rank;
    const A* gr = dkv + (a.own_kv ? a.kv_rank + a.rot : 0);
    float sq = 0.f;
    for (int i = threadIdx.x; i < a.q_rank; i += 256) {
        const float v = (float)dq[i];
        sq += v * v;
    }
    const float inv_q = 1.0f / sqrtf(block_sum_256(sq, red) / (float)a.q_rank + a.eps);
    A* cq = (A*)a.cq_out + t * a.q_rank;
    for (int i = threadIdx.x; i < a.q_rank; i += 256) cq[i] = (A)((float)dq[i] * inv_q * (float)((const A*)a.q_norm)[i]);
    if (a.gate_out)
        for (int h = threadIdx.x; h < a.H; h += 256) a.gate_out[t * a.H + h] = 1.0f / (1.0f + expf(-(float)gr[h]));
    if (!a.own_kv) return;
    const int64_t slot = a.slot_mapping ? a.slot_mapping[t] : -1;
    if (slot < 0) return;                                    // (uniform: a padded row)
    float sk = 0.f;
    for (int i = threadIdx.x; i < a.kv_rank; i += 256) {
        const float v = (float)dkv[i];
        sk += v * v;
    }
    const float inv_k = 1.0f / sqrtf(block_sum_256(sk, red) / (float)a.kv_rank + a.eps);
    A* kdst = (A*)a.k_cache + slot * (a.kv_rank + a.rot);
    A* vdst = (A*)a.v_cache + (slot / a.page) * a.page * a.kv_rank + slot % a.page;      // element i of the latent goes to vdst[i * page]
    for (int i = threadIdx.x; i < a.kv_rank; i += 256) {
        const A c = (A)((float)dkv[i] * inv_k * (float)((const A*)a.kv_norm)[i]);
        kdst[i] = c;
        vdst[(int64_t)i * a.page] = c;
    }
    const float pos = (float)a.positions[t];
    for (int d = threadIdx.x; d < a.rot; d += 256) {
        int partner, pair;
        bool first;
        pair_of(d, a.rot, a.interleaved, partner, pair, first);
        const float v = (float)dkv[a.kv_rank + d], o = (float)dkv[a.kv_rank + partner];
        float sn, cs;
        rot_sincos<A>(pos * a.freq[pair], sn, cs);
        const float c = cs * a.mag, s = sn * a.mag;
        kdst[a.kv_rank + d] = (A)(first ? v * c - o * s : v * c + o * s);
    }
}

// q [T, H, dim + rot] -> out[t, h, out_offset + d] = rotary(q[t, h, dim + d]), d < rot; out rows are [H, out_head] wide.
template <typename A>
__global__ __launch_bounds__(256) void latent_q_rotary_kernel(const A* __restrict__ q, int64_t q_stride, const int64_t* __restrict__ positions,
                                                              const float* __restrict__ freq, float mag, int interleaved, A* __restrict__ out,
                                                              int64_t out_stride, int H, int dim, int rot, int out_head, int out_offset) {
    const int64_t t = blockIdx.x;
    const float pos = (float)positions[t];
    for (int i = threadIdx.x; i < H * rot; i += 256) {
        const int h = i / rot, d = i - h * rot;
        int partner, pair;
        bool first;
        pair_of(d, rot, interleaved, partner, pair, first);
        const A* src = q + t * q_stride + (int64_t)h * (dim + rot) + dim;
        const float v = (float)src[d], o = (float)src[partner];
        float sn, cs;
        rot_sincos<A>(pos * freq[pair], sn, cs);
        const float c = cs * mag, s = sn * mag;
        out[t * out_stride + (int64_t)h * out_head + out_offset + d] = (A)(first ? v * c - o * s : v * c + o * s);
    }
}

struct HeadsArgs {
    const void* x;             // [M, ...]: head h's K inputs of row m start at x + m ldx + h x_head
    int64_t ldx, x_head;
    const void* w;             // [H, N, K]
    void* y;                   // head h's N outputs of row m start at y + m ldy + h y_head
    int64_t ldy, y_head;
    int M, N, K, vec_ok;
};

__global__ __launch_bounds__(256) void gemm_heads_bf16_kernel(HeadsArgs a) {
    const int h = blockIdx.z, m0 = blockIdx.y * nvh_any::GT;
    nvh_any::gemm_any_bf16_tile<false>((const bf16*)a.x + h * a.x_head, a.ldx, (const bf16*)a.w + (int64_t)h * a.N * a.K, a.K, nullptr, (bf16*)a.y + h * a.y_head, a.ldy,
                                       nvh_any::RowMap{nullptr, m0, min(nvh_any::GT, a.M - m0)}, blockIdx.x * nvh_any::GT, a.N, a.K, a.vec_ok);
}

__global__ __launch_bounds__(256) void gemm_heads_f32_kernel(HeadsArgs a) {
    const int h = blockIdx.z, m0 = blockIdx.y * nvh_any::GT;
    nvh_any::gemm_any_f32_tile((const float*)a.x + h * a.x_head, a.ldx, (const float*)a.w + (int64_t)h * a.N * a.K, a.K, nullptr, (float*)a.y + h * a.y_head, a.ldy,
                               nvh_any::RowMap{nullptr, m0, min(nvh_any::GT, a.M - m0)}, blockIdx.x * nvh_any::GT, a.N, a.K);
}

}  // namespace

extern "C" int32_t nvh_latent_prep(const void* proj, int64_t proj_row_stride, int64_t q_rank, int64_t kv_rank, int64_t rot_dim, int64_t heads, int32_t own_kv,
                                   const void* q_norm_weight, const void* kv_norm_weight, float eps, const int64_t* positions, const float* freq, float mag,
                                   int32_t interleaved, void* cq_out, float* gate_out, void* k_cache, void* v_cache, const int32_t* slot_mapping,
                                   int64_t page, int64_t num_tokens, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(proj && q_norm_weight && cq_out && positions, NVH_EINVAL, "nvh_latent_prep: null pointer");
    NVH_REQUIRE(!own_kv || (kv_norm_weight && k_cache && v_cache && slot_mapping && (rot_dim == 0 || freq)), NVH_EINVAL, "nvh_latent_prep: null pointer (key/value side)");
    NVH_REQUIRE(num_tokens >= 0 && q_rank > 0 && kv_rank > 0 && rot_dim >= 0 && rot_dim % 2 == 0 && heads > 0 && page > 0, NVH_EINVAL, "nvh_latent_prep: bad sizes");
    NVH_REQUIRE(proj_row_stride >= q_rank + (own_kv ? kv_rank + rot_dim : 0) + (gate_out ? heads : 0), NVH_EINVAL, "nvh_latent_prep: projection row too short");
    if (num_tokens == 0) return NVH_OK;
    const LatentPrepArgs a{proj, proj_row_stride, (int)q_rank, (int)kv_rank, (int)rot_dim, (int)heads, own_kv, q_norm_weight, kv_norm_weight, eps, positions, freq, mag,
                           interleaved, cq_out, gate_out, k_cache, v_cache, slot_mapping, (int)page};
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) latent_prep_kernel<float><<<dim3((unsigned)num_tokens), 256, 0, st>>>(a);
    else latent_prep_kernel<bf16><<<dim3((unsigned)num_tokens), 256, 0, st>>>(a);
    NVH_CHECK_LAUNCH("nvh_latent_prep");
    return NVH_OK;
}

extern "C" int32_t nvh_latent_q_rotary(const void* q, int64_t q_row_stride, const int64_t* positions, const float* freq, float mag, int32_t interleaved,
                                       void* out, int64_t out_row_stride, int64_t num_tokens, int64_t heads, int64_t dim, int64_t rot_dim,
                                       int64_t out_head_size, int64_t out_offset, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(q && positions && out && (rot_dim == 0 || freq), NVH_EINVAL, "nvh_latent_q_rotary: null pointer");
    NVH_REQUIRE(num_tokens >= 0 && heads > 0 && dim >= 0 && rot_dim >= 0 && rot_dim % 2 == 0 && out_offset >= 0 && out_offset + rot_dim <= out_head_size &&
                    q_row_stride >= heads * (dim + rot_dim) && out_row_stride >= heads * out_head_size,
                NVH_EINVAL, "nvh_latent_q_rotary: bad sizes");
    if (num_tokens == 0 || rot_dim == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) latent_q_rotary_kernel<float><<<dim3((unsigned)num_tokens), 256, 0, st>>>((const float*)q, q_row_stride, positions, freq, mag, interleaved, (float*)out, out_row_stride, (int)heads, (int)dim, (int)rot_dim, (int)out_head_size, (int)out_offset);
    else latent_q_rotary_kernel<bf16><<<dim3((unsigned)num_tokens), 256, 0, st>>>((const bf16*)q, q_row_stride, positions, freq, mag, interleaved, (bf16*)out, out_row_stride, (int)heads, (int)dim, (int)rot_dim, (int)out_head_size, (int)out_offset);
    NVH_CHECK_LAUNCH("nvh_latent_q_rotary");
    return NVH_OK;
}

extern "C" int32_t nvh_gemm_heads_nt(const void* x, int64_t x_row_stride, int64_t x_head_stride, const void* w, void* y, int64_t y_row_stride,
                                     int64_t y_head_stride, int64_t M, int64_t heads, int64_t N, int64_t K, int32_t act_f32, nvh_stream_t stream) {
    NVH_REQUIRE(x && w && y, NVH_EINVAL, "nvh_gemm_heads_nt: null pointer");
    NVH_REQUIRE(M >= 0 && heads > 0 && heads < 65536 && N > 0 && K > 0 && M < (1 << 22) && N < (1 << 30) && K < (1 << 30) && x_head_stride >= 0 && y_head_stride >= N &&
                    x_row_stride >= (heads - 1) * x_head_stride + K && y_row_stride >= (heads - 1) * y_head_stride + N,
                NVH_EINVAL, "nvh_gemm_heads_nt: bad sizes");
    if (M == 0) return NVH_OK;
    const int vec_ok = !act_f32 && K % 8 == 0 && x_row_stride % 8 == 0 && x_head_stride % 8 == 0 && nvh_aligned16(x) && nvh_aligned16(w);
    const HeadsArgs a{x, x_row_stride, x_head_stride, w, y, y_row_stride, y_head_stride, (int)M, (int)N, (int)K, vec_ok};
    const dim3 grid((unsigned)nvh_cdiv(N, nvh_any::GT), (unsigned)nvh_cdiv(M, nvh_any::GT), (unsigned)heads);
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) gemm_heads_f32_kernel<<<grid, 256, 0, st>>>(a);
    else gemm_heads_bf16_kernel<<<grid, 256, 0, st>>>(a);
    NVH_CHECK_LAUNCH("nvh_gemm_heads_nt");
    return NVH_OK;
}
