// Row-wise operators around an fp32 residual stream, for designs whose residual sum, norms and softcap must stay in
// 32-bit while projections run in the activation type A (bf16, or fp32 for a model served in full precision):
//   embedding rows -> fp32 stream (+ a copy in A), Dynamic-Tanh norm fused with the residual add that precedes it,
//   tanh-GELU gate, [stream | first embedding] concatenation for a looped stack, row gather, logit softcap.
// Every kernel is one workgroup per row (or a flat element grid) with 16-byte accesses where the row allows.
#include "common.h"
#include "gemm_any.h"

namespace {

template <typename A>
__device__ __forceinline__ float ldf(const A* p, int64_t i) {
    return (float)p[i];
}

struct DytNorm {            // tanh(alpha * x) * w + b; all three in the activation type
    const void* alpha;
    const void* w;
    const void* b;
};

// tanh for the norm: the library's where everything is fp32; for bf16 results 1 - 2 / (e^2z + 1) on the hardware's 2^x and
// reciprocal (about 1e-6 absolute; the result is rounded to 8 bits of mantissa).
template <typename A>
__device__ __forceinline__ float dyt_tanh(float z) {
    if constexpr (sizeof(A) == 4) {
        return tanhf(z);
    } else {
        const float e = __builtin_amdgcn_exp2f(fminf(z, 20.f) * 2.8853900817779268f);        // e^(2z)
        return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
    }
}

// x[row] = (accumulate ? x[row] : 0) + post(y[row]) + bias;  h[row] = next(x[row]).
// y null: the stream is only normalised.  post / next with a null weight are skipped (next: no h written).
// VEC: dim % 4 == 0 and every row 16-byte (A: 8-byte) aligned: four consecutive elements per lane, one access each.
template <typename A, bool VEC>
__global__ __launch_bounds__(256) void residual_dyt_kernel(const A* __restrict__ y, int64_t y_stride, DytNorm post, const A* __restrict__ bias,
                                                           float* __restrict__ x, int accumulate, DytNorm next, A* __restrict__ h,
                                                           int64_t h_stride, int dim) {
    typedef A A4 __attribute__((ext_vector_type(4)));
    const int64_t row = blockIdx.x;
    const float pa = post.w ? ldf((const A*)post.alpha, 0) : 0.f;
    const float na = next.w ? ldf((const A*)next.alpha, 0) : 0.f;
    float* xr = x + row * dim;
    constexpr int W = VEC ? 4 : 1;
    for (int c = threadIdx.x * W; c < dim; c += 256 * W) {
        float s[W], t[W], bv[W], pw[W], pb[W], nw[W], nb[W];
        if constexpr (VEC) {
            const f32x4 xv = accumulate ? *reinterpret_cast<const f32x4*>(xr + c) : f32x4{0.f, 0.f, 0.f, 0.f};
            const A4 zero = {(A)0.f, (A)0.f, (A)0.f, (A)0.f};
            const A4 yv = y ? *reinterpret_cast<const A4*>(y + row * y_stride + c) : zero;
            const A4 b4 = bias ? *reinterpret_cast<const A4*>(bias + c) : zero;
            const A4 pw4 = post.w ? *reinterpret_cast<const A4*>((const A*)post.w + c) : zero, pb4 = post.w ? *reinterpret_cast<const A4*>((const A*)post.b + c) : zero;
            const A4 nw4 = next.w ? *reinterpret_cast<const A4*>((const A*)next.w + c) : zero, nb4 = next.w ? *reinterpret_cast<const A4*>((const A*)next.b + c) : zero;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                s[e] = xv[e];
                t[e] = (float)yv[e];
                bv[e] = (float)b4[e];
                pw[e] = (float)pw4[e];
                pb[e] = (float)pb4[e];
                nw[e] = (float)nw4[e];
                nb[e] = (float)nb4[e];
            }
        } else {
            s[0] = accumulate ? xr[c] : 0.f;
            t[0] = y ? ldf(y, row * y_stride + c) : 0.f;
            bv[0] = bias ? ldf(bias, c) : 0.f;
            pw[0] = post.w ? ldf((const A*)post.w, c) : 0.f;
            pb[0] = post.w ? ldf((const A*)post.b, c) : 0.f;
            nw[0] = next.w ? ldf((const A*)next.w, c) : 0.f;
            nb[0] = next.w ? ldf((const A*)next.b, c) : 0.f;
        }
        float hv[W];
#pragma unroll
        for (int e = 0; e < W; ++e) {
            if (y) s[e] += post.w ? dyt_tanh<A>(pa * t[e]) * pw[e] + pb[e] : t[e];
            s[e] += bv[e];
            hv[e] = next.w ? dyt_tanh<A>(na * s[e]) * nw[e] + nb[e] : 0.f;
        }
        if constexpr (VEC) {
            if (y || bias) *reinterpret_cast<f32x4*>(xr + c) = f32x4{s[0], s[1], s[2], s[3]};
            if (next.w) *reinterpret_cast<A4*>(h + row * h_stride + c) = A4{(A)hv[0], (A)hv[1], (A)hv[2], (A)hv[3]};
        } else {
            if (y || bias) xr[c] = s[0];
            if (next.w) h[row * h_stride + c] = (A)hv[0];
        }
    }
}

template <typename A>
__global__ __launch_bounds__(256) void embedding_stream_kernel(const int64_t* __restrict__ ids, const A* __restrict__ table, float* __restrict__ x,
                                                               A* __restrict__ x0, int64_t x0_stride, int dim, int64_t vocab) {
    const int64_t row = blockIdx.x;
    const int64_t id = ids[row];
    const bool ok = id >= 0 && id < vocab;
    for (int c = threadIdx.x; c < dim; c += 256) {
        const A v = ok ? table[id * dim + c] : (A)0.f;
        x[row * dim + c] = (float)v;
        if (x0) x0[row * x0_stride + c] = v;
    }
}

// out[row, :dim] = A(x[row]); the second half of the row (the first embedding) is already there.
template <typename A>
__global__ __launch_bounds__(256) void stream_cast_kernel(const float* __restrict__ x, A* __restrict__ out, int64_t out_stride, int dim) {
    const int64_t row = blockIdx.x;
    for (int c = threadIdx.x; c < dim; c += 256) out[row * out_stride + c] = (A)x[row * dim + c];
}

template <typename A>
__global__ __launch_bounds__(256) void gelu_tanh_mul_kernel(const A* __restrict__ gu, int64_t gu_stride, A* __restrict__ y, int64_t rows, int inter) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * inter) return;
    const int64_t row = i / inter;
    const int c = (int)(i - row * inter);
    const float g = ldf(gu, row * gu_stride + c), u = ldf(gu, row * gu_stride + inter + c);
    const float act = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    y[i] = (A)(act * u);
}

__global__ __launch_bounds__(256) void gather_rows_f32_kernel(const float* __restrict__ x, const int32_t* __restrict__ index, float* __restrict__ out, int dim) {
    const int64_t row = blockIdx.x;
    const int64_t src = index[row];
    for (int c = threadIdx.x; c < dim; c += 256) out[row * dim + c] = x[src * dim + c];
}

template <typename A>
__global__ __launch_bounds__(256) void softcap_kernel(const A* __restrict__ z, int64_t z_stride, float* __restrict__ out, int64_t rows, int vocab, float cap) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * vocab) return;
    const int64_t row = i / vocab;
    const float v = ldf(z, row * z_stride + (i - row * vocab));
    out[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
}

// x[row] = table[id] * scale + pos_table[position] (fp32); ids or positions outside their tables give zeros for that term.
template <typename A>
__global__ __launch_bounds__(256) void embedding_pos_stream_kernel(const int64_t* __restrict__ ids, const int64_t* __restrict__ positions,
                                                                   const A* __restrict__ table, const A* __restrict__ pos_table, float scale,
                                                                   float* __restrict__ x, int dim, int64_t vocab, int64_t max_pos) {
    const int64_t row = blockIdx.x;
    const int64_t id = ids[row], p = pos_table ? positions[row] : -1;
    const bool ok = id >= 0 && id < vocab, pok = p >= 0 && p < max_pos;
    for (int c = threadIdx.x; c < dim; c += 256) {
        const float e = ok ? (float)table[id * dim + c] * scale : 0.f;
        x[row * dim + c] = e + (pok ? (float)pos_table[p * dim + c] : 0.f);
    }
}

__device__ __forceinline__ float block_sum4(float v, float* scratch) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    return scratch[0] + scratch[1] + scratch[2] + scratch[3];
}

// The close of a layer whose sublayers all read one norm of the stream, and the norm that opens the next layer, per row:
//   s = branch_scale * (unit(a) wa + unit(b) wb) + c + c32;   x <- x + s;   h <- norm(x)
// unit(v) = v / sqrt(mean(v^2) + branch_eps) where the branch has a weight (wa / wb), v itself where it has none; absent
// terms are skipped.  norm: 1 = layer norm ((x - mean) / sqrt(var + eps) w + b, var the mean squared deviation),
// 2 = RMS norm (x rsqrt(mean of squares + eps) w), 0 = none (no h).  Everything is fp32; the row sits in LDS meanwhile.
struct CloseArgs {
    const void *a, *wa, *b, *wb, *c;
    const float* c32;
    int64_t a_stride, b_stride, c_stride, c32_stride;
    float branch_scale, branch_eps;
    float* x;
    int norm;
    const void *nw, *nb;
    float eps;
    void* h;
    int64_t h_stride;
    int dim;
};

template <typename A>
__global__ __launch_bounds__(256) void residual_norm_kernel(CloseArgs p) {
    extern __shared__ float rowbuf[];
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const int dim = p.dim;
    const A* a = p.a ? (const A*)p.a + row * p.a_stride : nullptr;
    const A* b = p.b ? (const A*)p.b + row * p.b_stride : nullptr;
    const A* c = p.c ? (const A*)p.c + row * p.c_stride : nullptr;
    const float* c32 = p.c32 ? p.c32 + row * p.c32_stride : nullptr;
    float ia = 1.f, ib = 1.f;
    if (a && p.wa) {
        float s = 0.f;
        for (int i = threadIdx.x; i < dim; i += 256) {
            const float v = (float)a[i];
            s += v * v;
        }
        ia = 1.0f / sqrtf(block_sum4(s, red) / (float)dim + p.branch_eps);
    }
    if (b && p.wb) {
        float s = 0.f;
        for (int i = threadIdx.x; i < dim; i += 256) {
            const float v = (float)b[i];
            s += v * v;
        }
        ib = 1.0f / sqrtf(block_sum4(s, red) / (float)dim + p.branch_eps);
    }
    float* xr = p.x + row * dim;
    float sum = 0.f;
    for (int i = threadIdx.x; i < dim; i += 256) {
        float s = 0.f;
        if (a) s += p.wa ? (float)a[i] * ia * (float)((const A*)p.wa)[i] : (float)a[i];
        if (b) s += p.wb ? (float)b[i] * ib * (float)((const A*)p.wb)[i] : (float)b[i];
        s *= p.branch_scale;
        if (c) s += (float)c[i];
        if (c32) s += c32[i];
        const float v = xr[i] + s;
        if (a || b || c || c32) xr[i] = v;
        rowbuf[i] = v;
        sum += v;
    }
    if (p.norm == 0) return;
    float mean = 0.f;
    if (p.norm == 1) mean = block_sum4(sum, red) / (float)dim;
    float sq = 0.f;
    for (int i = threadIdx.x; i < dim; i += 256) {
        const float d = rowbuf[i] - mean;
        sq += d * d;
    }
    const float inv = 1.0f / sqrtf(block_sum4(sq, red) / (float)dim + p.eps);
    A* h = (A*)p.h + row * p.h_stride;
    for (int i = threadIdx.x; i < dim; i += 256) {
        float v = (rowbuf[i] - mean) * inv * (float)((const A*)p.nw)[i];
        if (p.nb) v += (float)((const A*)p.nb)[i];
        h[i] = (A)v;
    }
}

// The close of a sublayer in a stack that norms AFTER the sum, per row:
//   v = alpha x + ls (y + y32);   x <- v rsqrt(mean(v^2) + eps) (offset + w);   h <- x in the activation type
// alpha: the weight of the old stream in the sum; ls: a per-column scale of the sublayer's result (null: 1); y (type A) and
// y32 (fp32) are the sublayer's result, either or both may be absent (none: the norm alone, with alpha; write_x 0 then leaves
// the stream as it is and gives h only).  offset 1 serves
// a weight that is stored around zero.  The stream stays fp32; the sum, the statistics and the product are fp32.
struct PostNormArgs {
    const void* y;
    int64_t y_stride;
    const float* y32;
    int64_t y32_stride;
    const void* ls;
    float alpha;
    float* x;
    const void* nw;
    float offset, eps;
    void* h;
    int64_t h_stride;
    int dim, write_x;
};

template <typename A>
__global__ __launch_bounds__(256) void residual_postnorm_kernel(PostNormArgs p) {
    extern __shared__ float rowbuf[];
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const int dim = p.dim;
    const A* y = p.y ? (const A*)p.y + row * p.y_stride : nullptr;
    const float* y32 = p.y32 ? p.y32 + row * p.y32_stride : nullptr;
    const A* ls = (const A*)p.ls;
    float* xr = p.x + row * dim;
    float sq = 0.f;
    for (int i = threadIdx.x; i < dim; i += 256) {
        float v = p.alpha * xr[i];
        if (y || y32) {
            float s = y ? (float)y[i] : 0.f;
            if (y32) s += y32[i];
            if (ls) s *= (float)ls[i];
            v += s;
        }
        rowbuf[i] = v;
        sq += v * v;
    }
    const float inv = 1.0f / sqrtf(block_sum4(sq, red) / (float)dim + p.eps);
    A* h = p.h ? (A*)p.h + row * p.h_stride : nullptr;
    for (int i = threadIdx.x; i < dim; i += 256) {
        const float v = rowbuf[i] * inv * (p.offset + (float)((const A*)p.nw)[i]);
        if (p.write_x) xr[i] = v;
        if (h) h[i] = (A)v;
    }
}

// The close of a sublayer whose RESULT is normed before it joins the stream (the sublayer itself read the stream as it is), per row:
//   y = sa a + sb b + c32;   x <- x + mult * w * y / sqrt(mean(y^2) + eps);   h <- x in the activation type (when asked for)
// a, b (type A) and c32 (fp32) are the sublayer's terms, any of them absent; w: one number for all columns (w_elems 1) or one a
// column.  Sums, statistics and the stream are fp32; the row sits in LDS between the two passes.
struct SubNormArgs {
    const void *a, *b;
    const float* c32;
    int64_t a_stride, b_stride, c32_stride;
    float sa, sb, mult, eps;
    const void* w;
    int w_elems;
    float* x;
    void* h;
    int64_t h_stride;
    int dim;
};

template <typename A>
__global__ __launch_bounds__(256) void residual_subnorm_kernel(SubNormArgs p) {
    extern __shared__ float rowbuf[];
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const int dim = p.dim;
    const A* a = p.a ? (const A*)p.a + row * p.a_stride : nullptr;
    const A* b = p.b ? (const A*)p.b + row * p.b_stride : nullptr;
    const float* c32 = p.c32 ? p.c32 + row * p.c32_stride : nullptr;
    float sq = 0.f;
    for (int i = threadIdx.x; i < dim; i += 256) {
        float y = 0.f;
        if (a) y = p.sa * (float)a[i];
        if (b) y = __builtin_fmaf(p.sb, (float)b[i], y);
        if (c32) y += c32[i];
        rowbuf[i] = y;
        sq += y * y;
    }
    const float inv = p.mult / sqrtf(block_sum4(sq, red) / (float)dim + p.eps);
    float* xr = p.x + row * dim;
    A* h = p.h ? (A*)p.h + row * p.h_stride : nullptr;
    const A* w = (const A*)p.w;
    for (int i = threadIdx.x; i < dim; i += 256) {
        const float v = xr[i] + rowbuf[i] * inv * (float)w[p.w_elems == 1 ? 0 : i];
        xr[i] = v;
        if (h) h[i] = (A)v;
    }
}

// y = act(g) (* u when gated): g = columns [0, inter) and u = columns [inter, 2 inter) of the row.
// act: 0 silu, 1 gelu (tanh form), 2 squared relu.
template <typename A>
__global__ __launch_bounds__(256) void act_mul_kernel(const A* __restrict__ gu, int64_t gu_stride, A* __restrict__ y, int64_t y_stride, int64_t rows, int inter,
                                                      int act, int gated) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * inter) return;
    const int64_t row = i / inter;
    const int c = (int)(i - row * inter);
    const float g = ldf(gu, row * gu_stride + c);
    float v;
    if (act == 0) v = g / (1.0f + expf(-g));
    else if (act == 1) v = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    else v = g > 0.f ? g * g : 0.f;
    if (gated) v *= ldf(gu, row * gu_stride + inter + c);
    y[row * y_stride + c] = (A)v;
}

template <typename A>
__global__ __launch_bounds__(256) void logits_scale_kernel(const A* __restrict__ z, int64_t z_stride, float* __restrict__ out, int64_t rows, int vocab, float scale,
                                                           float cap) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * vocab) return;
    const int64_t row = i / vocab;
    const float v = ldf(z, row * z_stride + (i - row * vocab)) * scale;
    out[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
}


// ---------------------------------------------------------------------------------------------------------------
// The any-shape product (gemm_any.h) over one weight matrix: tile (blockIdx.x, blockIdx.y) covers 64 columns and the 64
// rows that start at 64 blockIdx.y.
template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_any_bf16_kernel(const bf16* __restrict__ x, int64_t ldx, const bf16* __restrict__ w, int64_t ldw,
                                                            const bf16* __restrict__ bias, void* __restrict__ yv, int64_t ldy, int M, int N, int K,
                                                            int vec_ok) {
    const int m0 = blockIdx.y * nvh_any::GT;
    nvh_any::gemm_any_bf16_tile<OUT_F32>(x, ldx, w, ldw, bias, yv, ldy, nvh_any::RowMap{nullptr, m0, min(nvh_any::GT, M - m0)}, blockIdx.x * nvh_any::GT, N, K, vec_ok);
}

__global__ __launch_bounds__(256) void gemm_any_f32_kernel(const float* __restrict__ x, int64_t ldx, const float* __restrict__ w, int64_t ldw,
                                                           const float* __restrict__ bias, float* __restrict__ y, int64_t ldy, int M, int N, int K) {
    const int m0 = blockIdx.y * nvh_any::GT;
    nvh_any::gemm_any_f32_tile(x, ldx, w, ldw, bias, y, ldy, nvh_any::RowMap{nullptr, m0, min(nvh_any::GT, M - m0)}, blockIdx.x * nvh_any::GT, N, K);
}

}  // namespace

#define NVH_STREAM_ARGS_OK(name, cond) NVH_REQUIRE(cond, NVH_EINVAL, name ": bad argument")

extern "C" int32_t nvh_embedding_stream(const int64_t* ids, const void* table, float* x, void* x0, int64_t x0_stride,
                                        int64_t num_tokens, int64_t dim, int64_t vocab, int32_t act_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_embedding_stream", ids && table && x && num_tokens >= 0 && dim > 0 && vocab > 0);
    if (num_tokens == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) embedding_stream_kernel<float><<<dim3((unsigned)num_tokens), 256, 0, st>>>(ids, (const float*)table, x, (float*)x0, x0_stride, (int)dim, vocab);
    else embedding_stream_kernel<bf16><<<dim3((unsigned)num_tokens), 256, 0, st>>>(ids, (const bf16*)table, x, (bf16*)x0, x0_stride, (int)dim, vocab);
    NVH_CHECK_LAUNCH("nvh_embedding_stream");
    return NVH_OK;
}

extern "C" int32_t nvh_residual_dyt(const void* y, int64_t y_stride, const void* post_alpha, const void* post_w, const void* post_b,
                                    const void* bias, float* x, int32_t accumulate, const void* next_alpha, const void* next_w,
                                    const void* next_b, void* h, int64_t h_stride, int64_t rows, int64_t dim, int32_t act_f32,
                                    nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_residual_dyt", x && rows >= 0 && dim > 0 && (!post_w || (post_alpha && post_b && y)) &&
                                               (!next_w || (next_alpha && next_b && h)) && (accumulate || y || bias));
    if (rows == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    const DytNorm post{post_alpha, post_w, post_b}, next{next_alpha, next_w, next_b};
    const int esz = act_f32 ? 4 : 2;
    auto al = [&](const void* p, int bytes) { return p == nullptr || ((uintptr_t)p % bytes) == 0; };
    const bool vec = dim % 4 == 0 && al(x, 16) && al(y, 4 * esz) && y_stride % 4 == 0 && al(h, 4 * esz) && h_stride % 4 == 0 && al(bias, 4 * esz) &&
                     al(post_w, 4 * esz) && al(post_b, 4 * esz) && al(next_w, 4 * esz) && al(next_b, 4 * esz);
    const dim3 grid((unsigned)rows);
    if (act_f32) {
        if (vec) residual_dyt_kernel<float, true><<<grid, 256, 0, st>>>((const float*)y, y_stride, post, (const float*)bias, x, accumulate, next, (float*)h, h_stride, (int)dim);
        else residual_dyt_kernel<float, false><<<grid, 256, 0, st>>>((const float*)y, y_stride, post, (const float*)bias, x, accumulate, next, (float*)h, h_stride, (int)dim);
    } else {
        if (vec) residual_dyt_kernel<bf16, true><<<grid, 256, 0, st>>>((const bf16*)y, y_stride, post, (const bf16*)bias, x, accumulate, next, (bf16*)h, h_stride, (int)dim);
        else residual_dyt_kernel<bf16, false><<<grid, 256, 0, st>>>((const bf16*)y, y_stride, post, (const bf16*)bias, x, accumulate, next, (bf16*)h, h_stride, (int)dim);
    }
    NVH_CHECK_LAUNCH("nvh_residual_dyt");
    return NVH_OK;
}

extern "C" int32_t nvh_stream_cast(const float* x, void* out, int64_t out_stride, int64_t rows, int64_t dim, int32_t act_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_stream_cast", x && out && rows >= 0 && dim > 0 && out_stride >= dim);
    if (rows == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) stream_cast_kernel<float><<<dim3((unsigned)rows), 256, 0, st>>>(x, (float*)out, out_stride, (int)dim);
    else stream_cast_kernel<bf16><<<dim3((unsigned)rows), 256, 0, st>>>(x, (bf16*)out, out_stride, (int)dim);
    NVH_CHECK_LAUNCH("nvh_stream_cast");
    return NVH_OK;
}

extern "C" int32_t nvh_gelu_tanh_mul(const void* gate_up, int64_t row_stride, void* y, int64_t rows, int64_t inter, int32_t act_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_gelu_tanh_mul", gate_up && y && rows >= 0 && inter > 0 && row_stride >= 2 * inter);
    if (rows == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    const unsigned blocks = (unsigned)nvh_cdiv(rows * inter, 256);
    if (act_f32) gelu_tanh_mul_kernel<float><<<dim3(blocks), 256, 0, st>>>((const float*)gate_up, row_stride, (float*)y, rows, (int)inter);
    else gelu_tanh_mul_kernel<bf16><<<dim3(blocks), 256, 0, st>>>((const bf16*)gate_up, row_stride, (bf16*)y, rows, (int)inter);
    NVH_CHECK_LAUNCH("nvh_gelu_tanh_mul");
    return NVH_OK;
}

extern "C" int32_t nvh_gather_rows_f32(const float* x, const int32_t* index, float* out, int64_t rows, int64_t dim, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_gather_rows_f32", x && index && out && rows >= 0 && dim > 0);
    if (rows == 0) return NVH_OK;
    gather_rows_f32_kernel<<<dim3((unsigned)rows), 256, 0, (hipStream_t)stream>>>(x, index, out, (int)dim);
    NVH_CHECK_LAUNCH("nvh_gather_rows_f32");
    return NVH_OK;
}

extern "C" int32_t nvh_logit_softcap(const void* logits, int64_t row_stride, float* out, int64_t rows, int64_t vocab, float cap, int32_t act_f32,
                                     nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_logit_softcap", logits && out && rows >= 0 && vocab > 0 && row_stride >= vocab);
    if (rows == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    const unsigned blocks = (unsigned)nvh_cdiv(rows * vocab, 256);
    if (act_f32) softcap_kernel<float><<<dim3(blocks), 256, 0, st>>>((const float*)logits, row_stride, out, rows, (int)vocab, cap);
    else softcap_kernel<bf16><<<dim3(blocks), 256, 0, st>>>((const bf16*)logits, row_stride, out, rows, (int)vocab, cap);
    NVH_CHECK_LAUNCH("nvh_logit_softcap");
    return NVH_OK;
}

extern "C" int32_t nvh_gemm_any_nt(const void* x, int64_t x_row_stride, const void* w, const void* bias, void* y, int64_t y_row_stride,
                                   int64_t M, int64_t N, int64_t K, int32_t in_f32, int32_t out_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_gemm_any_nt", x && w && y && M >= 0 && N > 0 && K > 0 && M < (1 << 30) && N < (1 << 30) && K < (1 << 30) &&
                                              x_row_stride >= K && y_row_stride >= N);
    NVH_REQUIRE(!in_f32 || out_f32, NVH_ENOSYS, "nvh_gemm_any_nt: fp32 operands give an fp32 product");
    if (M == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)nvh_cdiv(N, nvh_any::GT), (unsigned)nvh_cdiv(M, nvh_any::GT));
    if (in_f32) {
        gemm_any_f32_kernel<<<grid, 256, 0, st>>>((const float*)x, x_row_stride, (const float*)w, K, (const float*)bias, (float*)y, y_row_stride, (int)M, (int)N, (int)K);
    } else {
        const int vec_ok = K % 8 == 0 && x_row_stride % 8 == 0 && nvh_aligned16(x) && nvh_aligned16(w);
        if (out_f32) gemm_any_bf16_kernel<true><<<grid, 256, 0, st>>>((const bf16*)x, x_row_stride, (const bf16*)w, K, (const bf16*)bias, y, y_row_stride, (int)M, (int)N, (int)K, vec_ok);
        else gemm_any_bf16_kernel<false><<<grid, 256, 0, st>>>((const bf16*)x, x_row_stride, (const bf16*)w, K, (const bf16*)bias, y, y_row_stride, (int)M, (int)N, (int)K, vec_ok);
    }
    NVH_CHECK_LAUNCH("nvh_gemm_any_nt");
    return NVH_OK;
}

extern "C" int32_t nvh_embedding_pos_stream(const int64_t* ids, const int64_t* positions, const void* table, const void* pos_table, float scale,
                                            float* x, int64_t num_tokens, int64_t dim, int64_t vocab, int64_t max_positions, int32_t act_f32,
                                            nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_embedding_pos_stream", ids && table && x && num_tokens >= 0 && dim > 0 && vocab > 0 && (!pos_table || (positions && max_positions > 0)));
    if (num_tokens == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) embedding_pos_stream_kernel<float><<<dim3((unsigned)num_tokens), 256, 0, st>>>(ids, positions, (const float*)table, (const float*)pos_table, scale, x, (int)dim, vocab, max_positions);
    else embedding_pos_stream_kernel<bf16><<<dim3((unsigned)num_tokens), 256, 0, st>>>(ids, positions, (const bf16*)table, (const bf16*)pos_table, scale, x, (int)dim, vocab, max_positions);
    NVH_CHECK_LAUNCH("nvh_embedding_pos_stream");
    return NVH_OK;
}

extern "C" int32_t nvh_residual_norm(const void* a, int64_t a_stride, const void* a_weight, const void* b, int64_t b_stride, const void* b_weight,
                                     float branch_scale, float branch_eps, const void* c, int64_t c_stride, const float* c32, int64_t c32_stride,
                                     float* x, int32_t norm_kind, const void* norm_weight, const void* norm_bias, float eps, void* h, int64_t h_stride,
                                     int64_t rows, int64_t dim, int32_t act_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_residual_norm", x && rows >= 0 && dim > 0 && dim <= 32768 && norm_kind >= 0 && norm_kind <= 2 && (norm_kind == 0 || (norm_weight && h)) &&
                                                (!a_weight || a) && (!b_weight || b));
    if (rows == 0) return NVH_OK;
    const CloseArgs p{a, a_weight, b, b_weight, c, c32, a_stride, b_stride, c_stride, c32_stride, branch_scale, branch_eps, x, norm_kind,
                      norm_weight, norm_bias, eps, h, h_stride, (int)dim};
    hipStream_t st = (hipStream_t)stream;
    const size_t lds = sizeof(float) * (size_t)dim;
    if (lds > 48 * 1024) {
        const hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(&residual_norm_kernel<float>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        const hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(&residual_norm_kernel<bf16>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        NVH_REQUIRE(e1 == hipSuccess && e2 == hipSuccess, NVH_ENOSYS, "nvh_residual_norm: %zu bytes of LDS refused", lds);
    }
    if (act_f32) residual_norm_kernel<float><<<dim3((unsigned)rows), 256, lds, st>>>(p);
    else residual_norm_kernel<bf16><<<dim3((unsigned)rows), 256, lds, st>>>(p);
    NVH_CHECK_LAUNCH("nvh_residual_norm");
    return NVH_OK;
}

extern "C" int32_t nvh_residual_postnorm(const void* y, int64_t y_stride, const float* y32, int64_t y32_stride, const void* layer_scale, float alpha,
                                         float* x, int32_t write_x, const void* norm_weight, float weight_offset, float eps, void* h, int64_t h_stride,
                                         int64_t rows, int64_t dim, int32_t act_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_residual_postnorm", x && norm_weight && rows >= 0 && dim > 0 && dim <= 32768 && (!y || y_stride >= dim) && (!y32 || y32_stride >= dim) &&
                                                    (!h || h_stride >= dim));
    if (rows == 0) return NVH_OK;
    const PostNormArgs p{y, y_stride, y32, y32_stride, layer_scale, alpha, x, norm_weight, weight_offset, eps, h, h_stride, (int)dim, write_x};
    hipStream_t st = (hipStream_t)stream;
    const size_t lds = sizeof(float) * (size_t)dim;
    if (lds > 48 * 1024) {
        const hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(&residual_postnorm_kernel<float>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        const hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(&residual_postnorm_kernel<bf16>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        NVH_REQUIRE(e1 == hipSuccess && e2 == hipSuccess, NVH_ENOSYS, "nvh_residual_postnorm: %zu bytes of LDS refused", lds);
    }
    if (act_f32) residual_postnorm_kernel<float><<<dim3((unsigned)rows), 256, lds, st>>>(p);
    else residual_postnorm_kernel<bf16><<<dim3((unsigned)rows), 256, lds, st>>>(p);
    NVH_CHECK_LAUNCH("nvh_residual_postnorm");
    return NVH_OK;
}

extern "C" int32_t nvh_residual_subnorm(const void* a, int64_t a_stride, float a_scale, const void* b, int64_t b_stride, float b_scale, const float* c32,
                                        int64_t c32_stride, float mult, const void* weight, int64_t weight_elems, float eps, float* x, void* h,
                                        int64_t h_stride, int64_t rows, int64_t dim, int32_t act_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_residual_subnorm", x && weight && (a || b || c32) && rows >= 0 && dim > 0 && dim <= 32768 && (weight_elems == 1 || weight_elems == dim));
    if (rows == 0) return NVH_OK;
    const SubNormArgs p{a, b, c32, a_stride, b_stride, c32_stride, a_scale, b_scale, mult, eps, weight, (int)weight_elems, x, h, h_stride, (int)dim};
    hipStream_t st = (hipStream_t)stream;
    const size_t lds = sizeof(float) * (size_t)dim;
    if (lds > 48 * 1024) {
        const hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(&residual_subnorm_kernel<float>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        const hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(&residual_subnorm_kernel<bf16>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        NVH_REQUIRE(e1 == hipSuccess && e2 == hipSuccess, NVH_ENOSYS, "nvh_residual_subnorm: %zu bytes of LDS refused", lds);
    }
    if (act_f32) residual_subnorm_kernel<float><<<dim3((unsigned)rows), 256, lds, st>>>(p);
    else residual_subnorm_kernel<bf16><<<dim3((unsigned)rows), 256, lds, st>>>(p);
    NVH_CHECK_LAUNCH("nvh_residual_subnorm");
    return NVH_OK;
}

extern "C" int32_t nvh_act_mul(const void* x, int64_t row_stride, void* y, int64_t y_stride, int64_t rows, int64_t inter, int32_t act, int32_t gated,
                               int32_t act_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_act_mul", x && y && rows >= 0 && inter > 0 && act >= 0 && act <= 2 && row_stride >= (gated ? 2 : 1) * inter && y_stride >= inter);
    if (rows == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    const unsigned blocks = (unsigned)nvh_cdiv(rows * inter, 256);
    if (act_f32) act_mul_kernel<float><<<dim3(blocks), 256, 0, st>>>((const float*)x, row_stride, (float*)y, y_stride, rows, (int)inter, act, gated);
    else act_mul_kernel<bf16><<<dim3(blocks), 256, 0, st>>>((const bf16*)x, row_stride, (bf16*)y, y_stride, rows, (int)inter, act, gated);
    NVH_CHECK_LAUNCH("nvh_act_mul");
    return NVH_OK;
}

extern "C" int32_t nvh_logits_scale(const void* logits, int64_t row_stride, float* out, int64_t rows, int64_t vocab, float scale, float cap,
                                    int32_t act_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_logits_scale", logits && out && rows >= 0 && vocab > 0 && row_stride >= vocab);
    if (rows == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    const unsigned blocks = (unsigned)nvh_cdiv(rows * vocab, 256);
    if (act_f32) logits_scale_kernel<float><<<dim3(blocks), 256, 0, st>>>((const float*)logits, row_stride, out, rows, (int)vocab, scale, cap);
    else logits_scale_kernel<bf16><<<dim3(blocks), 256, 0, st>>>((const bf16*)logits, row_stride, out, rows, (int)vocab, scale, cap);
    NVH_CHECK_LAUNCH("nvh_logits_scale");
    return NVH_OK;
}
