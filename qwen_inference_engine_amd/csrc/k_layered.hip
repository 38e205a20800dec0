// k_layered.hip — kernels of the layered-model engine tier (engine_layered.hip): the
// mechanisms that the Qwen decoder does not have, each with its constants as parameters.
//
//   lay::linear            y = A W^T, fp32 accumulation in k order; A fp32 (optionally rounded to
//                          bf16 on load), W fp32 or bf16; batched (per head) and grouped (per
//                          expert) forms
//   lay::latent_post       latent KV: RMS norm of the compressed row, rotate-half rotary of the
//                          shared key part and of every head's rotated query part, paged append
//   lay::latent_attention  sliding-window attention over the latent cache in absorbed form
//                          (scores against [c ; k_rot], output in latent space), online softmax
//   lay::head_gate         per-head sigmoid output gate
//   lay::postnorm_add      y = x + g * v / sqrt(mean(v^2) + eps): a branch's result is normed, then added
//   lay::depth_mix         x = sum_j a[j] X_j over the stack of earlier layer results
//   lay::route_topk, moe_group, moe_gather, moe_combine: sigmoid router whose score scales the
//                          expert's input, or biased logits whose softmax over the chosen ones
//                          weights the outputs; rows grouped by expert for the grouped linear
//   lay::silu_mul, embed_rows, final_rows, rows_to_bf16
//
// Everything the residual stream, a norm, a router, a score or a softmax touches is fp32.  No
// result depends on which other rows are in the launch: every output element is reduced in an
// order fixed by its own sizes.
#include "k_layered.hpp"

namespace qie {
namespace lay {

template <typename T> __device__ __forceinline__ float ldf(const T* p, int64_t i);
template <> __device__ __forceinline__ float ldf<float>(const float* p, int64_t i) { return p[i]; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p, int64_t i) { return bf2f(p[i]); }
template <typename T> __device__ __forceinline__ void stf(T* p, int64_t i, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, int64_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, int64_t i, float v) { p[i] = f2bf(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
// block-wide sum over 256 threads (4 waves); every thread gets the result
__device__ __forceinline__ float block_sum256(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// ------------------------------------------------------------------ linear
constexpr int LBM = 64, LBN = 64, LBK = 16;

template <typename TW>
__global__ __launch_bounds__(256) void linear_kernel(LinearP p) {
    __shared__ float As[LBK][LBM + 4];
    __shared__ float Ws[LBK][LBN + 4];
    const int z = blockIdx.z;
    int m_lo = 0, m_hi = p.M;
    if (p.grp_off) {
        m_lo = p.grp_off[z];
        m_hi = p.grp_off[z + 1];
    }
    const int m0 = m_lo + blockIdx.y * LBM;
    if (m0 >= m_hi) return;
    const int n0 = blockIdx.x * LBN;
    const float* A = p.A + (int64_t)z * p.sA;
    const TW* W = (const TW*)p.W + (int64_t)z * p.sW;
    float* Y = p.Y + (int64_t)z * p.sY;
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < p.K; k0 += LBK) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int idx = tid + i * 256, r = idx >> 4, kk = idx & 15;
            const int m = m0 + r, n = n0 + r, k = k0 + kk;
            float a = 0.f, w = 0.f;
            if (k < p.K) {
                if (m < m_hi) {
                    a = A[(int64_t)m * p.lda + k];
                    if (p.round_a) a = rbf(a);
                }
                if (n < p.N) w = ldf<TW>(W, (int64_t)n * p.ldw + k);
            }
            As[kk][r] = a;
            Ws[kk][r] = w;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < LBK; kk++) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                a[i] = As[kk][ty * 4 + i];
                w[i] = Ws[kk][tx * 4 + i];
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int m = m0 + ty * 4 + i;
        if (m >= m_hi) continue;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int n = n0 + tx * 4 + j;
            if (n < p.N) Y[(int64_t)m * p.ldy + n] = acc[i][j];
        }
    }
}

// Few rows (decoding, or few rows per expert): one wave per output column streams the weight
// row once with 16-byte loads and keeps up to 16 rows' sums in registers, so the launch is as
// wide as N x batch whatever M is.  VEC: K, the row strides and the batch strides keep every
// 8-element run aligned; else one element per lane and step.
template <typename TW, bool VEC>
__global__ __launch_bounds__(256) void linear_skinny_kernel(LinearP p) {
    const int z = blockIdx.z, lane = threadIdx.x & 63;
    const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
    int m_lo = 0, m_hi = p.M;
    if (p.grp_off) {
        m_lo = p.grp_off[z];
        m_hi = p.grp_off[z + 1];
    }
    const int m0 = m_lo + blockIdx.y * 16;
    if (m0 >= m_hi || n >= p.N) return;
    const int rows = min(16, m_hi - m0);
    const float* A = p.A + (int64_t)z * p.sA + (int64_t)m0 * p.lda;
    const TW* W = (const TW*)p.W + (int64_t)z * p.sW + (int64_t)n * p.ldw;
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
    if (VEC) {
        for (int k = lane * 8; k < p.K; k += 512) {
            float w[8];
            if (sizeof(TW) == 2) {
                const uint4 u = *reinterpret_cast<const uint4*>((const uint16_t*)W + k);
                w[0] = bf_lo(u.x); w[1] = bf_hi(u.x); w[2] = bf_lo(u.y); w[3] = bf_hi(u.y);
                w[4] = bf_lo(u.z); w[5] = bf_hi(u.z); w[6] = bf_lo(u.w); w[7] = bf_hi(u.w);
            } else {
                const float4 u0 = *reinterpret_cast<const float4*>((const float*)W + k);
                const float4 u1 = *reinterpret_cast<const float4*>((const float*)W + k + 4);
                w[0] = u0.x; w[1] = u0.y; w[2] = u0.z; w[3] = u0.w; w[4] = u1.x; w[5] = u1.y; w[6] = u1.z; w[7] = u1.w;
            }
#pragma unroll
            for (int i = 0; i < 16; i++) {
                if (i < rows) {
                    const float4 a0 = *reinterpret_cast<const float4*>(A + (int64_t)i * p.lda + k);
                    const float4 a1 = *reinterpret_cast<const float4*>(A + (int64_t)i * p.lda + k + 4);
                    float a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
                    float t = 0.f;
#pragma unroll
                    for (int j = 0; j < 8; j++) t = fmaf(p.round_a ? rbf(a[j]) : a[j], w[j], t);
                    acc[i] += t;
                }
            }
        }
    } else {
        for (int k = lane; k < p.K; k += 64) {
            const float w = ldf<TW>(W, k);
#pragma unroll
            for (int i = 0; i < 16; i++)
                if (i < rows) {
                    const float a = A[(int64_t)i * p.lda + k];
                    acc[i] = fmaf(p.round_a ? rbf(a) : a, w, acc[i]);
                }
        }
    }
    float* Y = p.Y + (int64_t)z * p.sY + (int64_t)m0 * p.ldy + n;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float v = wave_sum(acc[i]);
        if (lane == 0 && i < rows) Y[(int64_t)i * p.ldy] = v;
    }
}

// Many rows, bf16 weights, batched (per head) or grouped (per expert): MFMA tiles straight from
// memory.  A wave owns 16 rows x 64 columns; per 32 k it converts its A rows (fp32, 8 per lane)
// to one bf16 fragment and multiplies it with 4 weight fragments (16 bytes per lane each, the
// rows of W are the columns of the product).  The 4 waves of a workgroup take 64 rows against
// the same columns, so the weight fragments meet in the L1.  K a multiple of 8; k beyond K has a
// zero A fragment; rows / columns beyond the range read a valid row again and are not stored.
typedef __bf16 lbf16x8_t __attribute__((ext_vector_type(8)));
typedef float lf32x4_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void linear_mfma_kernel(LinearP p) {
    const int z = blockIdx.z, lane = threadIdx.x & 63, g = lane >> 4, n = lane & 15;
    int m_lo = 0, m_hi = p.M;
    if (p.grp_off) {
        m_lo = p.grp_off[z];
        m_hi = p.grp_off[z + 1];
    }
    const int m0 = m_lo + blockIdx.y * 64 + (threadIdx.x >> 6) * 16;
    if (m0 >= m_hi) return;
    const int n0 = blockIdx.x * 64;
    const int mr = min(m0 + n, m_hi - 1);
    const float* A = p.A + (int64_t)z * p.sA + (int64_t)mr * p.lda;
    const uint16_t* W = (const uint16_t*)p.W + (int64_t)z * p.sW;
    const uint16_t* wr[4];
#pragma unroll
    for (int c = 0; c < 4; c++) wr[c] = W + (int64_t)min(n0 + 16 * c + n, p.N - 1) * p.ldw;
    lf32x4_t acc[4];
#pragma unroll
    for (int c = 0; c < 4; c++) acc[c] = lf32x4_t{0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < p.K; k0 += 32) {
        const int k = k0 + 8 * g;
        const bool in = k < p.K;
        const int kc = in ? k : 0;
        const float4 a0 = *reinterpret_cast<const float4*>(A + kc);
        const float4 a1 = *reinterpret_cast<const float4*>(A + kc + 4);
        uint4 wv[4];
#pragma unroll
        for (int c = 0; c < 4; c++) wv[c] = *reinterpret_cast<const uint4*>(wr[c] + kc);
        uint4 af = make_uint4(pack2(a0.x, a0.y), pack2(a0.z, a0.w), pack2(a1.x, a1.y), pack2(a1.z, a1.w));
        if (!in) af = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
        for (int c = 0; c < 4; c++)
            acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lbf16x8_t, af), __builtin_bit_cast(lbf16x8_t, wv[c]),
                                                             acc[c], 0, 0, 0);
    }
    // lane holds rows m0 + 4 g + j, column n0 + 16 c + n
    float* Y = p.Y + (int64_t)z * p.sY;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const int col = n0 + 16 * c + n;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int m = m0 + 4 * g + j;
            if (m < m_hi && col < p.N) Y[(int64_t)m * p.ldy + col] = acc[c][j];
        }
    }
}

static bool al16p(const void* q) { return ((uintptr_t)q & 15) == 0; }

int linear(const LinearP& p, bool w_f32, hipStream_t st) {
    QIE_REQUIRE(p.A && p.W && p.Y && p.M > 0 && p.N > 0 && p.K > 0 && p.batch > 0, "layered linear: bad arguments");
    const bool a_vec = p.lda % 4 == 0 && p.sA % 4 == 0 && al16p(p.A);
    if (p.M <= 32) {
        const bool vec = a_vec && p.K % 8 == 0 && p.ldw % 8 == 0 && p.sW % 8 == 0 && al16p(p.W);
        dim3 grid((unsigned)((p.N + 3) / 4), (unsigned)((p.M + 15) / 16), (unsigned)p.batch);
        if (w_f32) {
            if (vec) hipLaunchKernelGGL((linear_skinny_kernel<float, true>), grid, dim3(256), 0, st, p);
            else hipLaunchKernelGGL((linear_skinny_kernel<float, false>), grid, dim3(256), 0, st, p);
        } else {
            if (vec) hipLaunchKernelGGL((linear_skinny_kernel<uint16_t, true>), grid, dim3(256), 0, st, p);
            else hipLaunchKernelGGL((linear_skinny_kernel<uint16_t, false>), grid, dim3(256), 0, st, p);
        }
        QIE_LAUNCH_CHECK();
        return 0;
    }
    if (!w_f32 && p.round_a && p.mfma && a_vec && p.K % 8 == 0 && p.ldw % 8 == 0 && p.sW % 8 == 0 && al16p(p.W)) {
        dim3 grid((unsigned)((p.N + 63) / 64), (unsigned)((p.M + 63) / 64), (unsigned)p.batch);
        hipLaunchKernelGGL(linear_mfma_kernel, grid, dim3(256), 0, st, p);
        QIE_LAUNCH_CHECK();
        return 0;
    }
    dim3 grid((unsigned)((p.N + LBN - 1) / LBN), (unsigned)((p.M + LBM - 1) / LBM), (unsigned)p.batch);
    if (w_f32)
        hipLaunchKernelGGL(linear_kernel<float>, grid, dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL(linear_kernel<uint16_t>, grid, dim3(256), 0, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ embedding rows
// out[t] = E[tok[t]] * scale (+ the sinusoidal vector of the row's position when pos: entry 2i =
// sin(pos * freq[i]), entry 2i + 1 = cos of the same; freq and the angle in double, rounded once)
template <typename TW>
__global__ __launch_bounds__(256) void embed_rows_kernel(const TW* E, const int32_t* tok, float* out, uint16_t* out_bf, int W,
                                                         int vocab, float scale, const int32_t* pos, const double* freq) {
    const int t = blockIdx.x;
    int id = tok[t];
    if (id < 0 || id >= vocab) id = 0;
    if (pos) {   // a thread takes the pairs (2i, 2i + 1): one sine and cosine of the pair's angle
        const double p = (double)pos[t];
        for (int i = threadIdx.x; 2 * i < W; i += 256) {
            double sn, cs;
            sincos(p * freq[i], &sn, &cs);
            const int w = 2 * i;
            const float v0 = ldf<TW>(E, (int64_t)id * W + w) * scale + (float)sn;
            out[(int64_t)t * W + w] = v0;
            if (out_bf) out_bf[(int64_t)t * W + w] = f2bf(v0);
            if (w + 1 < W) {
                const float v1 = ldf<TW>(E, (int64_t)id * W + w + 1) * scale + (float)cs;
                out[(int64_t)t * W + w + 1] = v1;
                if (out_bf) out_bf[(int64_t)t * W + w + 1] = f2bf(v1);
            }
        }
        return;
    }
    for (int w = threadIdx.x; w < W; w += 256) {
        const float v = ldf<TW>(E, (int64_t)id * W + w) * scale;
        out[(int64_t)t * W + w] = v;
        if (out_bf) out_bf[(int64_t)t * W + w] = f2bf(v);
    }
}
int embed_rows(const void* E, bool w_f32, const int32_t* tok, float* out, uint16_t* out_bf, int T, int W, int vocab,
               hipStream_t st, float scale, const int32_t* pos, const double* freq) {
    QIE_REQUIRE(!pos || freq, "embed_rows: positions without their frequencies");
    if (w_f32)
        hipLaunchKernelGGL(embed_rows_kernel<float>, dim3(T), dim3(256), 0, st, (const float*)E, tok, out, out_bf, W, vocab, scale, pos,
                           freq);
    else
        hipLaunchKernelGGL(embed_rows_kernel<uint16_t>, dim3(T), dim3(256), 0, st, (const uint16_t*)E, tok, out, out_bf, W, vocab,
                           scale, pos, freq);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ latent post-projection
// One block per row.  proj row = [q (H x (dim + rot)) | c (R) | k_rot (rot) | ...].  The rotary
// pairs coordinate i with i + dims/2 inside the first `dims` coordinates of a rotated part.
__device__ __forceinline__ const void* latent_row(const LatentCache& c, int slot, int pos, int64_t layer_off, int D,
                                                  int elem) {
    const int page = c.table[(int64_t)slot * c.max_pages + pos / c.page_tokens];
    const int64_t e = (int64_t)page * c.page_stride + layer_off + (int64_t)(pos % c.page_tokens) * D;
    return (const char*)c.pool + e * elem;
}

template <typename TC>
__global__ __launch_bounds__(256) void latent_post_kernel(LatentPostP p) {
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int slot = p.row_slot[t], pos = p.row_pos[t];
    float* row = p.proj + (int64_t)t * p.ld;
    const int half = p.rot_dims / 2;
    const float* cs = p.rope_cos + (int64_t)pos * half;
    const float* sn = p.rope_sin + (int64_t)pos * half;
    const int hq = p.dim + p.rot;
    // queries: rotate the rotated part of every head in place; pair j is (j, j + half) or (2j, 2j + 1)
    const int ia = p.rot_layout ? 2 : 1, ib = p.rot_layout ? 1 : half;
    for (int i = tid; i < p.heads * half; i += 256) {
        const int h = i / half, j = i % half;
        float* q = row + h * hq + p.dim;
        const float u = q[j * ia], v = q[j * ia + ib];
        q[j * ia] = u * cs[j] - v * sn[j];
        q[j * ia + ib] = v * cs[j] + u * sn[j];
    }
    if (!p.own_kv) return;
    const float* d = p.kv ? p.kv + (int64_t)t * p.kv_ld : row + p.heads * hq;
    float ss = 0.f;
    for (int i = tid; i < p.R; i += 256) ss += d[i] * d[i];
    ss = block_sum256(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)p.R + p.eps);
    TC* out = (TC*)latent_row(p.cache, slot, pos, p.layer_off, p.R + p.rot, sizeof(TC));
    for (int i = tid; i < p.R; i += 256) stf<TC>(out, i, d[i] * inv * p.norm_w[i]);
    if (p.interleaved) {
        // second copy of c for the value product of the matrix-core attention: the 4 keys of a
        // group side by side for every latent coordinate
        const int pt = pos % p.cache.page_tokens;
        TC* region = out - (int64_t)pt * (p.R + p.rot);
        TC* ct = region + (int64_t)p.cache.page_tokens * (p.R + p.rot) + (int64_t)(pt >> 2) * p.R * 4 + (pt & 3);
        for (int i = tid; i < p.R; i += 256) stf<TC>(ct, (int64_t)i * 4, d[i] * inv * p.norm_w[i]);
    }
    const float* kr = d + p.R;
    for (int j = tid; j < p.rot; j += 256) {
        float v;
        if (j >= p.rot_dims)
            v = kr[j];
        else if (p.rot_layout)
            v = (j & 1) ? kr[j] * cs[j >> 1] + kr[j - 1] * sn[j >> 1] : kr[j] * cs[j >> 1] - kr[j + 1] * sn[j >> 1];
        else if (j < half)
            v = kr[j] * cs[j] - kr[j + half] * sn[j];
        else
            v = kr[j] * cs[j - half] + kr[j - half] * sn[j - half];
        stf<TC>(out, p.R + j, v);
    }
}
int latent_post(const LatentPostP& p, bool cache_f32, int T, hipStream_t st) {
    QIE_REQUIRE(p.rot_dims % 2 == 0 && p.rot_dims <= p.rot, "latent_post: rotary dims %d must be even and <= %d", p.rot_dims,
                p.rot);
    if (cache_f32)
        hipLaunchKernelGGL(latent_post_kernel<float>, dim3(T), dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL(latent_post_kernel<uint16_t>, dim3(T), dim3(256), 0, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ latent attention
// One block per (head, row).  The query in latent space q' = [W_uk,h^T q_nope ; q_rot] (D = R +
// rot floats) is scored against the cached rows [c_j ; k_rot_j] of positions
// max(0, pos - window + 1) .. pos; the output is sum_j p_j c_j (R floats), expanded by W_uv
// afterwards.  Keys go through in chunks of ATT_CHUNK with a running max and sum.
constexpr int ATT_CHUNK = 256;
constexpr int ATT_MAXR = 4;   // R <= 256 * ATT_MAXR

template <typename TC>
__global__ __launch_bounds__(256) void latent_attention_kernel(LatentAttnP p) {
    extern __shared__ float sm[];
    float* q = sm;                  // [D]
    float* sc = sm + p.R + p.rot;   // [ATT_CHUNK]
    __shared__ float red[4];
    const int h = blockIdx.x, t = blockIdx.y, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int slot = p.row_slot[t], pos = p.row_pos[t];
    const int D = p.R + p.rot;
    const float* qa = p.q_abs + ((int64_t)t * p.heads + h) * p.R;
    const float* qr = p.proj + (int64_t)t * p.ld + h * (p.dim + p.rot) + p.dim;
    for (int i = tid; i < D; i += 256) q[i] = i < p.R ? qa[i] : qr[i - p.R];
    __syncthreads();
    int lo = pos - p.window + 1;
    if (lo < 0) lo = 0;
    float m_run = -INFINITY, l_run = 0.f;
    float acc[ATT_MAXR] = {};
    for (int j0 = lo; j0 <= pos; j0 += ATT_CHUNK) {
        const int nk = min(ATT_CHUNK, pos + 1 - j0);
        for (int jj = wave; jj < nk; jj += 4) {
            const TC* k = (const TC*)latent_row(p.cache, slot, j0 + jj, p.layer_off, D, sizeof(TC));
            float s = 0.f;
            for (int i = lane; i < D; i += 64) s = fmaf(q[i], ldf<TC>(k, i), s);
            s = wave_sum(s);
            if (lane == 0) sc[jj] = s * p.scale;
        }
        __syncthreads();
        float mx = -INFINITY;
        for (int jj = tid; jj < nk; jj += 256) mx = fmaxf(mx, sc[jj]);
        mx = wave_max(mx);
        if (lane == 0) red[wave] = mx;
        __syncthreads();
        mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        const float m_new = fmaxf(m_run, mx);
        const float alpha = expf(m_run - m_new);   // 0 on the first chunk
        __syncthreads();
        float ls = 0.f;
        for (int jj = tid; jj < nk; jj += 256) {
            const float e = expf(sc[jj] - m_new);
            sc[jj] = e;
            ls += e;
        }
        ls = block_sum256(ls, red);
        l_run = l_run * alpha + ls;
        m_run = m_new;
#pragma unroll
        for (int i = 0; i < ATT_MAXR; i++) acc[i] *= alpha;
        for (int jj = 0; jj < nk; jj++) {
            const TC* c = (const TC*)latent_row(p.cache, slot, j0 + jj, p.layer_off, D, sizeof(TC));
            const float w = sc[jj];
#pragma unroll
            for (int i = 0; i < ATT_MAXR; i++) {
                const int r = tid + i * 256;
                if (r < p.R) acc[i] = fmaf(w, ldf<TC>(c, r), acc[i]);
            }
        }
        __syncthreads();
    }
    const float inv = 1.0f / l_run;
    float* o = p.out + ((int64_t)t * p.heads + h) * p.R;
#pragma unroll
    for (int i = 0; i < ATT_MAXR; i++) {
        const int r = tid + i * 256;
        if (r < p.R) o[r] = acc[i] * inv;
    }
}
int latent_attention(const LatentAttnP& p, bool cache_f32, int T, hipStream_t st) {
    QIE_REQUIRE(p.R <= 256 * ATT_MAXR, "latent attention: latent size %d above %d", p.R, 256 * ATT_MAXR);
    QIE_REQUIRE(p.window >= 1, "latent attention: window %d", p.window);
    const size_t shm = (size_t)(p.R + p.rot + ATT_CHUNK) * 4;
    if (cache_f32)
        hipLaunchKernelGGL(latent_attention_kernel<float>, dim3(p.heads, T), dim3(256), shm, st, p);
    else
        hipLaunchKernelGGL(latent_attention_kernel<uint16_t>, dim3(p.heads, T), dim3(256), shm, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ per-head output gate
// v[t, h, :] *= sigmoid(gate[t, h]); gate logits sit in the projection row at column g_col
__global__ __launch_bounds__(256) void head_gate_kernel(float* v, uint16_t* v_bf, const float* proj, int64_t ld, int g_col, int heads,
                                                        int vd, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int64_t t = i / ((int64_t)heads * vd);
    const int h = (int)((i / vd) % heads);
    const float g = proj[t * ld + g_col + h];
    const float o = v[i] * (1.0f / (1.0f + expf(-g)));
    v[i] = o;
    if (v_bf) v_bf[i] = f2bf(o);
}
int head_gate(float* v, uint16_t* v_bf, const float* proj, int64_t ld, int g_col, int heads, int vd, int T, hipStream_t st) {
    const int64_t n = (int64_t)T * heads * vd;
    hipLaunchKernelGGL(head_gate_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, v, v_bf, proj, ld, g_col, heads, vd, n);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ norm on the sublayer output
__global__ __launch_bounds__(256) void postnorm_add_kernel(const float* x, const float* v, float* y, uint16_t* y_bf, int W,
                                                           float gain, float eps) {
    __shared__ float red[4];
    const int64_t t = blockIdx.x;
    float ss = 0.f;
    for (int i = threadIdx.x; i < W; i += 256) {
        const float a = v[t * W + i];
        ss += a * a;
    }
    ss = block_sum256(ss, red);
    const float inv = gain / sqrtf(ss / (float)W + eps);
    for (int i = threadIdx.x; i < W; i += 256) {
        const float o = (x ? x[t * W + i] : 0.f) + v[t * W + i] * inv;
        y[t * W + i] = o;
        if (y_bf) y_bf[t * W + i] = f2bf(o);
    }
}
int postnorm_add(const float* x, const float* v, float* y, uint16_t* y_bf, int T, int W, float gain, float eps, hipStream_t st) {
    hipLaunchKernelGGL(postnorm_add_kernel, dim3(T), dim3(256), 0, st, x, v, y, y_bf, W, gain, eps);
    QIE_LAUNCH_CHECK();
    return 0;
}

// rows picked by index, normed with one gain: out[i] = gain * x[rows[i]] / rms
__global__ __launch_bounds__(256) void final_rows_kernel(const float* x, const int32_t* rows, float* out, uint16_t* out_bf, int W,
                                                         float gain, const float* w1p, float eps, float w_one) {
    __shared__ float red[4];
    const int64_t t = rows[blockIdx.x];
    float ss = 0.f;
    for (int i = threadIdx.x; i < W; i += 256) {
        const float a = x[t * W + i];
        ss += a * a;
    }
    ss = block_sum256(ss, red);
    const float inv = gain / sqrtf(ss / (float)W + eps);
    for (int i = threadIdx.x; i < W; i += 256) {
        const float o = x[t * W + i] * inv * (w1p ? w_one + w1p[i] : 1.0f);
        out[(int64_t)blockIdx.x * W + i] = o;
        if (out_bf) out_bf[(int64_t)blockIdx.x * W + i] = f2bf(o);
    }
}
int final_rows(const float* x, const int32_t* rows, float* out, uint16_t* out_bf, int n, int W, float gain, const float* w1p,
               float eps, hipStream_t st, float w_one) {
    hipLaunchKernelGGL(final_rows_kernel, dim3(n), dim3(256), 0, st, x, rows, out, out_bf, W, gain, w1p, eps, w_one);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ depth-weighted average
// x[t, w] = sum_{j < n} a[j] X[j][t, w]; X[j] at stack + j * stride
__global__ __launch_bounds__(256) void depth_mix_kernel(const float* stack, int64_t stride, const float* a, int n, float* x,
                                                        uint16_t* x_bf, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    float s = 0.f;
    for (int j = 0; j < n; j++) s = fmaf(a[j], stack[j * stride + i], s);
    x[i] = s;
    if (x_bf) x_bf[i] = f2bf(s);
}
int depth_mix(const float* stack, int64_t stride, const float* a, int n, float* x, uint16_t* x_bf, int64_t count, hipStream_t st) {
    hipLaunchKernelGGL(depth_mix_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, st, stack, stride, a, n, x, x_bf,
                       count);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ gated activation
// a[m, j] = silu(gu[m, j]) * gu[m, ff + j]
// (act 1: the tanh form of gelu instead of silu, gelu(g) = g / 2 (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3))))
__global__ __launch_bounds__(256) void silu_mul_kernel(const float* gu, float* a, uint16_t* a_bf, int ff, int64_t n, int act) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int64_t m = i / ff;
    const int j = (int)(i % ff);
    const float g = gu[m * 2 * ff + j], u = gu[m * 2 * ff + ff + j];
    const float o = (act == 1 ? 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) : g / (1.0f + expf(-g))) * u;
    a[i] = o;
    if (a_bf) a_bf[i] = f2bf(o);
}
int silu_mul(const float* gu, float* a, uint16_t* a_bf, int64_t M, int ff, hipStream_t st, int act) {
    const int64_t n = M * ff;
    if (n == 0) return 0;
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, gu, a, a_bf, ff, n, act);
    QIE_LAUNCH_CHECK();
    return 0;
}

// a = xielu(u): ap u^2 + u / 2 for u > 0, else aq (exp(u) - 1 - u) + u / 2 (ap = softplus(p),
// aq = 1/2 + softplus(q), made once on the host)
__global__ __launch_bounds__(256) void xielu_kernel(const float* u, float* a, uint16_t* a_bf, float ap, float aq, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float z = u[i];
    const float o = z > 0.f ? fmaf(ap * z, z, 0.5f * z) : fmaf(aq, expm1f(z) - z, 0.5f * z);
    a[i] = o;
    if (a_bf) a_bf[i] = f2bf(o);
}
int xielu(const float* u, float* a, uint16_t* a_bf, int64_t n, float ap, float aq, hipStream_t st) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(xielu_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, u, a, a_bf, ap, aq, n);
    QIE_LAUNCH_CHECK();
    return 0;
}

// One wave's dot product of a row y [W] (fp32) with a weight row w [W]: 8 elements per lane and turn
// through 16-byte loads when W is a multiple of 8 (rows then start 16-byte aligned), else one
// element per lane and turn.  The order of the sum depends on W alone.
template <typename TW> __device__ __forceinline__ float wave_row_dot(const float* y, const TW* w, int W, int lane);
template <> __device__ __forceinline__ float wave_row_dot<uint16_t>(const float* y, const uint16_t* w, int W, int lane) {
    float z = 0.f;
    if ((W & 7) == 0) {
#pragma unroll 4
        for (int i = lane * 8; i < W; i += 512) {
            const uint4 u = *reinterpret_cast<const uint4*>(w + i);
            const float4 a = *reinterpret_cast<const float4*>(y + i), b = *reinterpret_cast<const float4*>(y + i + 4);
            z = fmaf(a.x, bf2f(u.x & 0xffffu), z);
            z = fmaf(a.y, bf2f(u.x >> 16), z);
            z = fmaf(a.z, bf2f(u.y & 0xffffu), z);
            z = fmaf(a.w, bf2f(u.y >> 16), z);
            z = fmaf(b.x, bf2f(u.z & 0xffffu), z);
            z = fmaf(b.y, bf2f(u.z >> 16), z);
            z = fmaf(b.z, bf2f(u.w & 0xffffu), z);
            z = fmaf(b.w, bf2f(u.w >> 16), z);
        }
    } else {
        for (int i = lane; i < W; i += 64) z = fmaf(y[i], bf2f(w[i]), z);
    }
    return wave_sum(z);
}
template <> __device__ __forceinline__ float wave_row_dot<float>(const float* y, const float* w, int W, int lane) {
    float z = 0.f;
    if ((W & 3) == 0) {
#pragma unroll 4
        for (int i = lane * 4; i < W; i += 256) {
            const float4 a = *reinterpret_cast<const float4*>(y + i), b = *reinterpret_cast<const float4*>(w + i);
            z = fmaf(a.x, b.x, z);
            z = fmaf(a.y, b.y, z);
            z = fmaf(a.z, b.z, z);
            z = fmaf(a.w, b.w, z);
        }
    } else {
        for (int i = lane; i < W; i += 64) z = fmaf(y[i], w[i], z);
    }
    return wave_sum(z);
}

// ------------------------------------------------------------------ mixture of experts
// Router: z = W_r y in fp32, s = sigmoid(z); the `top` largest (ties: the lower index) in
// descending order -> sel[t, k], score[t, k].  The ranking compares z, which orders the experts
// as s does but does not saturate (sigmoid(z) is 1.0f for every z above ~17).  One block per row.
template <typename TW>
__global__ __launch_bounds__(256) void route_kernel(const float* y, const TW* Wr, const float* bias, int W, int E, int top, int mode,
                                                    int32_t* sel, float* score) {
    extern __shared__ float s[];   // [E] router logits
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int e = wave; e < E; e += 4) {
        const float z = wave_row_dot<TW>(y + t * W, Wr + (int64_t)e * W, W, lane);
        if (lane == 0) s[e] = bias ? z + bias[e] : z;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float z0 = 0.f, den = 0.f;
        for (int k = 0; k < top; k++) {
            int best = -1;
            float bv = 0.f;
            for (int e = 0; e < E; e++)
                if (s[e] != -INFINITY && (best < 0 || s[e] > bv)) {
                    bv = s[e];
                    best = e;
                }
            if (best < 0) best = 0;   // only if logits are not finite
            sel[t * top + k] = best;
            if (mode == 0) {
                score[t * top + k] = 1.0f / (1.0f + expf(-bv));
            } else {   // softmax over the chosen logits: the first chosen is the largest
                if (k == 0) z0 = bv;
                const float ex = expf(bv - z0);
                score[t * top + k] = ex;
                den += ex;
            }
            s[best] = -INFINITY;
        }
        if (mode != 0)
            for (int k = 0; k < top; k++) score[t * top + k] /= den;
    }
}
int route_topk(const float* y, const void* Wr, const float* bias, bool w_f32, int T, int W, int E, int top, int mode, int32_t* sel,
               float* score, hipStream_t st) {
    QIE_REQUIRE(top >= 1 && top <= E && E <= 8192, "router: top %d of %d experts", top, E);
    if (w_f32)
        hipLaunchKernelGGL(route_kernel<float>, dim3(T), dim3(256), (size_t)E * 4, st, y, (const float*)Wr, bias, W, E, top, mode,
                           sel, score);
    else
        hipLaunchKernelGGL(route_kernel<uint16_t>, dim3(T), dim3(256), (size_t)E * 4, st, y, (const uint16_t*)Wr, bias, W, E, top,
                           mode, sel, score);
    QIE_LAUNCH_CHECK();
    return 0;
}

// Router over all E outputs (real and identity experts alike): s = softmax(z) in fp32; the choice
// ranks s + corr; a group of E / groups neighbours ranks by its largest choice score and only the
// `keep` best groups stay eligible (the others are excluded from the choice); the `top` best eligible
// are chosen, weighted by s / (sum of the chosen s + 1e-20) * scale.  Ties: the lower index.
// One block per row; shared: s [E], choice [E], group rank [groups].
template <typename TW>
__global__ __launch_bounds__(256) void route_grouped_kernel(const float* y, const TW* Wr, const float* corr, int W, int E, int top,
                                                            int groups, int keep, float scale, int32_t* sel, float* score) {
    extern __shared__ float sh[];
    float* s = sh;
    float* ch = sh + E;
    float* gs = ch + E;
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int e = wave; e < E; e += 4) {
        const float z = wave_row_dot<TW>(y + t * W, Wr + (int64_t)e * W, W, lane);
        if (lane == 0) s[e] = z;
    }
    __syncthreads();
    if (threadIdx.x != 0) return;
    float mx = s[0];
    for (int e = 1; e < E; e++) mx = fmaxf(mx, s[e]);
    float den = 0.f;
    for (int e = 0; e < E; e++) {
        s[e] = expf(s[e] - mx);
        den += s[e];
    }
    for (int e = 0; e < E; e++) {
        s[e] = s[e] / den;
        ch[e] = s[e] + corr[e];
    }
    const int per = E / groups;
    for (int g = 0; g < groups; g++) {
        float b = ch[g * per];
        for (int e = 1; e < per; e++) b = fmaxf(b, ch[g * per + e]);
        gs[g] = b;
    }
    for (int g = 0; g < groups; g++) {   // a group stays when fewer than `keep` groups rank before it
        int before = 0;
        for (int o = 0; o < groups; o++) before += (gs[o] > gs[g]) || (gs[o] == gs[g] && o < g);
        if (before >= keep)
            for (int e = 0; e < per; e++) ch[g * per + e] = -INFINITY;
    }
    float sum = 0.f;
    for (int k = 0; k < top; k++) {
        int best = -1;
        float bv = 0.f;
        for (int e = 0; e < E; e++)
            if (ch[e] != -INFINITY && (best < 0 || ch[e] > bv)) {
                bv = ch[e];
                best = e;
            }
        if (best < 0) best = 0;   // only if scores are not finite
        sel[t * top + k] = best;
        score[t * top + k] = s[best];
        sum += s[best];
        ch[best] = -INFINITY;
    }
    const float inv = scale / (sum + 1e-20f);
    for (int k = 0; k < top; k++) score[t * top + k] *= inv;
}
int route_grouped(const float* y, const void* Wr, const float* corr, bool w_f32, int T, int W, int E, int top, int groups, int keep,
                  float scale, int32_t* sel, float* score, hipStream_t st) {
    QIE_REQUIRE(top >= 1 && top <= E && E <= 4096 && corr, "router: top %d of %d outputs", top, E);
    QIE_REQUIRE(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups && top <= keep * (E / groups),
                "router: %d groups of %d outputs, %d kept, top %d", groups, E, keep, top);
    const size_t shm = (size_t)(2 * E + groups) * 4;
    if (w_f32)
        hipLaunchKernelGGL(route_grouped_kernel<float>, dim3(T), dim3(256), shm, st, y, (const float*)Wr, corr, W, E, top, groups, keep,
                           scale, sel, score);
    else
        hipLaunchKernelGGL(route_grouped_kernel<uint16_t>, dim3(T), dim3(256), shm, st, y, (const uint16_t*)Wr, corr, W, E, top,
                           groups, keep, scale, sel, score);
    QIE_LAUNCH_CHECK();
    return 0;
}

// Grouping: entries i = t * top + k in index order, gathered per expert.  cnt[e] first, then
// off[e] = sum of the counts before e and slot_of[i] = off[sel[i]] + rank of i among its expert's.
__global__ __launch_bounds__(256) void moe_count_kernel(const int32_t* sel, int n, int32_t* cnt) {
    __shared__ int red[4];
    const int e = blockIdx.x;
    int c = 0;
    for (int i = threadIdx.x; i < n; i += 256) c += sel[i] == e;
    for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) cnt[e] = red[0] + red[1] + red[2] + red[3];
}
__global__ __launch_bounds__(256) void moe_fill_kernel(const int32_t* sel, int n, const int32_t* cnt, int E, int32_t* off,
                                                       int32_t* slot_of) {
    __shared__ int wsum[4];
    __shared__ int base_s;
    const int e = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    if (tid == 0) {
        int o = 0;
        for (int i = 0; i < e; i++) o += cnt[i];
        base_s = o;
        off[e] = o;
        if (e == E - 1) off[E] = o + cnt[e];
    }
    __syncthreads();
    int base = base_s;
    for (int i0 = 0; i0 < n; i0 += 256) {
        const int i = i0 + tid;
        const bool f = i < n && sel[i] == e;
        const unsigned long long b = __ballot(f);
        const int before = __popcll(b & ((1ull << lane) - 1ull));
        if (lane == 0) wsum[wave] = __popcll(b);
        __syncthreads();
        int wb = 0;
        for (int w = 0; w < wave; w++) wb += wsum[w];
        if (f) slot_of[i] = base + wb + before;
        base += wsum[0] + wsum[1] + wsum[2] + wsum[3];
        __syncthreads();
    }
}
int moe_group(const int32_t* sel, int n, int E, int32_t* cnt, int32_t* off, int32_t* slot_of, hipStream_t st) {
    hipLaunchKernelGGL(moe_count_kernel, dim3(E), dim3(256), 0, st, sel, n, cnt);
    QIE_LAUNCH_CHECK();
    hipLaunchKernelGGL(moe_fill_kernel, dim3(E), dim3(256), 0, st, sel, n, cnt, E, off, slot_of);
    QIE_LAUNCH_CHECK();
    return 0;
}
// xg[slot_of[i], :] = score[i] * y[i / top, :]
__global__ __launch_bounds__(256) void moe_gather_kernel(const float* y, const float* score, const int32_t* slot_of, int top, int W,
                                                         float* xg, uint16_t* xg_bf) {
    const int64_t i = blockIdx.x;
    const int64_t t = i / top, d = slot_of[i];
    const float s = score ? score[i] : 1.0f;
    for (int w = threadIdx.x; w < W; w += 256) {
        const float o = s * y[t * W + w];
        xg[d * W + w] = o;
        if (xg_bf) xg_bf[d * W + w] = f2bf(o);
    }
}
int moe_gather(const float* y, const float* score, const int32_t* slot_of, int T, int top, int W, float* xg, uint16_t* xg_bf,
               hipStream_t st) {
    hipLaunchKernelGGL(moe_gather_kernel, dim3(T * top), dim3(256), 0, st, y, score, slot_of, top, W, xg, xg_bf);
    QIE_LAUNCH_CHECK();
    return 0;
}
// f[t, :] = sum_k (score[t * top + k] or 1) * yd[slot_of[t * top + k], :]; a chosen expert >= n_real (when
// sel) is an identity expert: its output is the row's input y[t, :]
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* yd, const int32_t* slot_of, const float* score, int top, int W,
                                                          float* f, const int32_t* sel, int n_real, const float* y) {
    const int64_t t = blockIdx.x;
    for (int w = threadIdx.x; w < W; w += 256) {
        float s = 0.f;
        if (sel)
            for (int k = 0; k < top; k++) {
                const float o = sel[t * top + k] >= n_real ? y[t * W + w] : yd[(int64_t)slot_of[t * top + k] * W + w];
                s = fmaf(score ? score[t * top + k] : 1.0f, o, s);
            }
        else if (score)
            for (int k = 0; k < top; k++) s = fmaf(score[t * top + k], yd[(int64_t)slot_of[t * top + k] * W + w], s);
        else
            for (int k = 0; k < top; k++) s += yd[(int64_t)slot_of[t * top + k] * W + w];
        f[t * W + w] = s;
    }
}
int moe_combine(const float* yd, const int32_t* slot_of, const float* score, int T, int top, int W, float* f, hipStream_t st,
                const int32_t* sel, int n_real, const float* y) {
    QIE_REQUIRE(!sel || y, "moe_combine: identity experts need the rows' input");
    hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, st, yd, slot_of, score, top, W, f, sel, n_real, y);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ greedy choice on fp32 rows
// ids[m] = the index of the largest logit of row m (ties: the lowest index).  One block per row.
__global__ __launch_bounds__(256) void argmax_rows_kernel(const float* x, int64_t V, int32_t* ids) {
    __shared__ float bv[256];
    __shared__ int bi[256];
    const float* r = x + (int64_t)blockIdx.x * V;
    float v = -INFINITY;
    int idx = 0x7fffffff;
    for (int64_t i = threadIdx.x; i < V; i += 256)
        if (r[i] > v) {
            v = r[i];
            idx = (int)i;
        }
    bv[threadIdx.x] = v;
    bi[threadIdx.x] = idx;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) {
            const float w = bv[threadIdx.x + o];
            const int j = bi[threadIdx.x + o];
            if (w > bv[threadIdx.x] || (w == bv[threadIdx.x] && j < bi[threadIdx.x])) {
                bv[threadIdx.x] = w;
                bi[threadIdx.x] = j;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) ids[blockIdx.x] = bi[0] == 0x7fffffff ? 0 : bi[0];
}
int argmax_rows(const float* x, int M, int64_t V, int32_t* ids, hipStream_t st) {
    hipLaunchKernelGGL(argmax_rows_kernel, dim3(M), dim3(256), 0, st, x, V, ids);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ conversions
__global__ __launch_bounds__(256) void rows_to_bf16_kernel(const float* x, uint16_t* y, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = f2bf(x[i]);
}
int rows_to_bf16(const float* x, uint16_t* y, int64_t n, hipStream_t st) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(rows_to_bf16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, x, y, n);
    QIE_LAUNCH_CHECK();
    return 0;
}
// y[m, k] = bf16(x[m, k]) for M rows of K values with row strides ldx / ldy
__global__ __launch_bounds__(256) void rows_to_bf16_strided_kernel(const float* x, int64_t ldx, uint16_t* y, int64_t ldy, int K,
                                                                   int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int64_t m = i / K;
    const int k = (int)(i % K);
    y[m * ldy + k] = f2bf(x[m * ldx + k]);
}
int rows_to_bf16_strided(const float* x, int64_t ldx, uint16_t* y, int64_t ldy, int64_t M, int K, hipStream_t st) {
    const int64_t n = M * K;
    if (n == 0) return 0;
    hipLaunchKernelGGL(rows_to_bf16_strided_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, x, ldx, y, ldy, K, n);
    QIE_LAUNCH_CHECK();
    return 0;
}
__global__ __launch_bounds__(256) void bf16_to_f32_kernel(const uint16_t* x, float* y, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = bf2f(x[i]);
}
int bf16_to_f32(const uint16_t* x, float* y, int64_t n, hipStream_t st) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(bf16_to_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, x, y, n);
    QIE_LAUNCH_CHECK();
    return 0;
}

}  // namespace lay
}  // namespace qie
