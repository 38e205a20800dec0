// k_mixers.hip — mixers of the layered engine tier beside the latent attention (k_layered.hpp):
//
//   lay::gqa_post        q / k head norms, rotary (either pairing, partial), values turned by
//                        their position or taken from the raw keys, paged K / V append
//   lay::gqa_attention   grouped-query softmax attention over the paged rows with a causal,
//                        sliding or block-local mask and an optional log-distance bias; the
//                        weighted sum of turned values is turned back
//                        and / or a linear one with a slope per head; softmax weights (optionally with a
//                        sink: one more term exp(sink_h) in the denominator, no key, no value), or sigmoid
//                        weights with a bias per head; an optional sigmoid gate per head or per coordinate;
//                        bias vectors on q and k (gqa_post)
//   lay::gated_scan      gated linear recurrence with an fp32 state per slot and head
//   lay::mingru_scan     minGRU: a recurrence per channel, update gate and candidate from the current input alone
//   lay::head_norm_rows  per-head RMS norm with a weight
//   lay::add_norm        residual add of a normed branch fused with the next branch's input norm
//
// Scores, softmax statistics, norms, gates and the recurrent state are fp32; cache rows are
// fp32 or bf16 by the engine's compute type.  A row's result depends only on its own slot,
// position and cache rows, never on what else the launch holds.
#include "k_layered.hpp"

namespace qie {
namespace lay {

namespace {

template <typename T> __device__ __forceinline__ float ldc(const T* p, int64_t i);
template <> __device__ __forceinline__ float ldc<float>(const float* p, int64_t i) { return p[i]; }
template <> __device__ __forceinline__ float ldc<uint16_t>(const uint16_t* p, int64_t i) { return bf2f(p[i]); }
template <typename T> __device__ __forceinline__ void stc(T* p, int64_t i, float v);
template <> __device__ __forceinline__ void stc<float>(float* p, int64_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void stc<uint16_t>(uint16_t* p, int64_t i, float v) { p[i] = f2bf(v); }

__device__ __forceinline__ float wsum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wmax(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float bsum256(float v, float* red) {
    v = wsum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// Coordinate i of `buf` after the turn by the angles whose cos / sin are cs / sn (one per pair);
// only the first `dims` coordinates turn.  The pair (u, w) becomes (u c - w s, w c + u s);
// sign = -1 turns back.
__device__ __forceinline__ float turned(const float* buf, int i, int dims, int layout, const float* cs, const float* sn, float sign) {
    if (i >= dims) return buf[i];
    int j, partner;
    float sg;
    if (layout == 1) {
        j = i >> 1;
        partner = i ^ 1;
        sg = (i & 1) ? 1.f : -1.f;
    } else {
        const int half = dims >> 1;
        if (i < half) {
            j = i;
            partner = i + half;
            sg = -1.f;
        } else {
            j = i - half;
            partner = j;
            sg = 1.f;
        }
    }
    return buf[i] * cs[j] + sg * sign * buf[partner] * sn[j];
}

__device__ __forceinline__ int64_t page_base(const LatentCache& c, int slot, int pos) {
    const int page = c.table[(int64_t)slot * c.max_pages + pos / c.page_tokens];
    return (int64_t)page * c.page_stride;
}

}  // namespace

// ------------------------------------------------------------------ post-projection
// One block per row; a wave per head, the head's coordinates staged in LDS so that either pairing
// finds its partner.
template <typename TC>
__global__ __launch_bounds__(256) void gqa_post_kernel(GqaPostP p) {
    extern __shared__ float sm[];
    const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int slot = p.row_slot[t], pos = p.row_pos[t];
    const int mx = max(p.dim, p.vdim);
    float* buf = sm + wave * mx;
    float* row = p.proj + (int64_t)t * p.ld;
    const int64_t pb = page_base(p.cache, slot, pos);
    const int pt = pos % p.cache.page_tokens;
    const int H = p.heads, G = p.kv_heads, dim = p.dim, vdim = p.vdim;
    TC* krow = (TC*)p.cache.pool + pb + p.k_off + (int64_t)pt * G * dim;
    // value coordinate i of key head g: row-major rows, or one column of the page's transposed block
    TC* vbase = (TC*)p.cache.pool + pb + p.v_off;
    const int PT = p.cache.page_tokens;
    auto vidx = [&](int g, int i) -> int64_t {
        return p.v_transposed ? ((int64_t)g * vdim + i) * PT + pt : ((int64_t)pt * G + g) * vdim + i;
    };
    const float* cs = p.rope_cos + (int64_t)pos * (p.rot_dims / 2);
    const float* sn = p.rope_sin + (int64_t)pos * (p.rot_dims / 2);
    for (int h0 = 0; h0 < H + G; h0 += 4) {
        const int hh = h0 + wave;
        const bool on = hh < H + G, is_q = hh < H;
        float* x = row + (is_q ? p.q_col + hh * dim : p.k_col + (hh - H) * dim);
        const float* bias = !on ? nullptr : is_q ? (p.q_bias ? p.q_bias + hh * dim : nullptr) : (p.k_bias ? p.k_bias + (hh - H) * dim : nullptr);
        if (on) {
            float ss = 0.f;
            for (int i = lane; i < dim; i += 64) {
                const float a = bias ? x[i] + bias[i] : x[i];
                buf[i] = a;
                ss += a * a;
            }
            ss = wsum(ss);
            if (!is_q && p.v_col < 0)   // the value is the key as projected
                for (int i = lane; i < dim; i += 64) stc<TC>(vbase, vidx(hh - H, i), buf[i]);
            if (p.qk_norm) {
                const float inv = 1.0f / sqrtf(ss / (float)dim + p.eps);
                const float* w = p.qk_norm == 1 ? (is_q ? p.qn_w : p.kn_w) : nullptr;
                for (int i = lane; i < dim; i += 64) buf[i] = buf[i] * inv * (w ? w[i] : 1.0f);
            }
            if (is_q && p.q_temp_every > 0) {
                const float tq = 1.0f + p.q_temp_coef * logf((float)((pos + 1) / p.q_temp_every + 1));
                for (int i = lane; i < dim; i += 64) buf[i] *= tq;
            }
        }
        __syncthreads();
        if (on)
            for (int i = lane; i < dim; i += 64) {
                const float o = turned(buf, i, p.rot_dims, p.rot_layout, cs, sn, 1.f);
                if (is_q)
                    x[i] = o;
                else
                    stc<TC>(krow, (int64_t)(hh - H) * dim + i, o);
            }
        __syncthreads();
    }
    if (p.v_col < 0) return;
    const float* vcs = p.rot_values ? p.vrope_cos + (int64_t)pos * (vdim / 2) : nullptr;
    const float* vsn = p.rot_values ? p.vrope_sin + (int64_t)pos * (vdim / 2) : nullptr;
    for (int g0 = 0; g0 < G; g0 += 4) {
        const int g = g0 + wave;
        const bool on = g < G;
        if (on)
            for (int i = lane; i < vdim; i += 64) buf[i] = row[p.v_col + g * vdim + i];
        __syncthreads();
        if (on)
            for (int i = lane; i < vdim; i += 64)
                stc<TC>(vbase, vidx(g, i), p.rot_values ? turned(buf, i, vdim, p.rot_layout, vcs, vsn, 1.f) : buf[i]);
        __syncthreads();
    }
}

int gqa_post(const GqaPostP& p, bool cache_f32, int T, hipStream_t st) {
    QIE_REQUIRE(p.heads > 0 && p.kv_heads > 0 && p.heads % p.kv_heads == 0, "gqa_post: %d query heads over %d key heads", p.heads,
                p.kv_heads);
    QIE_REQUIRE(p.rot_dims % 2 == 0 && p.rot_dims <= p.dim, "gqa_post: rotary dims %d must be even and <= %d", p.rot_dims, p.dim);
    QIE_REQUIRE(!p.rot_values || p.vdim % 2 == 0, "gqa_post: turned values need an even vdim (%d)", p.vdim);
    QIE_REQUIRE(p.v_col >= 0 || p.vdim == p.dim, "gqa_post: keys as values need vdim == dim");
    const size_t shm = (size_t)4 * std::max(p.dim, p.vdim) * 4;
    QIE_REQUIRE(shm <= 48 * 1024, "gqa_post: head size %d above the kernel's staging", std::max(p.dim, p.vdim));
    if (cache_f32)
        hipLaunchKernelGGL(gqa_post_kernel<float>, dim3(T), dim3(256), shm, st, p);
    else
        hipLaunchKernelGGL(gqa_post_kernel<uint16_t>, dim3(T), dim3(256), shm, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ attention, exact form
// One block per (head, row): the visible keys go through in chunks of GA_CHUNK with a running
// maximum and sum; a wave scores a key, a thread owns value coordinates.
constexpr int GA_CHUNK = 256;
constexpr int GA_MAXV = 4;   // vdim <= 256 * GA_MAXV

__device__ __forceinline__ int first_visible(int mask, int size, int pos) {
    if (mask == 1) return max(0, pos - size + 1);
    if (mask == 2) return pos / size * size;
    return 0;
}

template <typename TC>
__global__ __launch_bounds__(256) void gqa_attention_kernel(GqaAttnP p) {
    extern __shared__ float sm[];
    float* q = sm;                 // [dim]
    float* sc = sm + p.dim;        // [GA_CHUNK]
    float* ob = sc + GA_CHUNK;     // [vdim]
    __shared__ float red[4];
    const int h = blockIdx.x, t = blockIdx.y, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int slot = p.row_slot[t], pos = p.row_pos[t];
    const int dim = p.dim, vdim = p.vdim, G = p.kv_heads, g = h / (p.heads / G);
    const float* qr = p.proj + (int64_t)t * p.ld + p.q_col + h * dim;
    for (int i = tid; i < dim; i += 256) q[i] = qr[i];
    __syncthreads();
    const int lo = first_visible(p.mask, p.mask_size, pos);
    const float b1 = p.r1 ? p.r1[h] : 0.f, b2 = p.r1 ? p.r2[h] : 0.f;
    const float slope = p.slopes ? p.slopes[h] : 0.f;
    const bool sig = p.pb != nullptr;
    const float pbh = sig ? p.pb[h] : 0.f;
    // a sink is a score without key or value: the running maximum and sum start from it
    float m_run = p.sink ? p.sink[h] : -INFINITY, l_run = p.sink ? 1.f : 0.f;
    float acc[GA_MAXV] = {};
    for (int j0 = lo; j0 <= pos; j0 += GA_CHUNK) {
        const int nk = min(GA_CHUNK, pos + 1 - j0);
        for (int jj = wave; jj < nk; jj += 4) {
            const int j = j0 + jj;
            const TC* k = (const TC*)p.cache.pool + page_base(p.cache, slot, j) + p.k_off +
                          ((int64_t)(j % p.cache.page_tokens) * G + g) * dim;
            float s = 0.f;
            for (int i = lane; i < dim; i += 64) s = fmaf(q[i], ldc<TC>(k, i), s);
            s = wsum(s);
            if (lane == 0) {
                s *= p.scale;
                if (p.r1) s -= b1 * log1pf(b2 * (float)(pos - j));
                if (p.slopes) s -= slope * (float)(pos - j);
                sc[jj] = sig ? 1.0f / (1.0f + expf(-(s + pbh))) : s;
            }
        }
        __syncthreads();
        if (sig) {   // the weights are final: no running maximum, no normalisation
            for (int jj = 0; jj < nk; jj++) {
                const int j = j0 + jj;
                const int pt = j % p.cache.page_tokens;
                const TC* v = (const TC*)p.cache.pool + page_base(p.cache, slot, j) + p.v_off;
                const float w = sc[jj];
#pragma unroll
                for (int i = 0; i < GA_MAXV; i++) {
                    const int r = tid + i * 256;
                    if (r < vdim)
                        acc[i] = fmaf(w, ldc<TC>(v, p.v_transposed ? ((int64_t)g * vdim + r) * p.cache.page_tokens + pt
                                                                     : ((int64_t)pt * G + g) * vdim + r), acc[i]);
                }
            }
            __syncthreads();
            continue;
        }
        float mx = -INFINITY;
        for (int jj = tid; jj < nk; jj += 256) mx = fmaxf(mx, sc[jj]);
        mx = wmax(mx);
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
        ls = bsum256(ls, red);
        l_run = l_run * alpha + ls;
        m_run = m_new;
#pragma unroll
        for (int i = 0; i < GA_MAXV; i++) acc[i] *= alpha;
        for (int jj = 0; jj < nk; jj++) {
            const int j = j0 + jj;
            const int pt = j % p.cache.page_tokens;
            const TC* v = (const TC*)p.cache.pool + page_base(p.cache, slot, j) + p.v_off;
            const float w = sc[jj];
#pragma unroll
            for (int i = 0; i < GA_MAXV; i++) {
                const int r = tid + i * 256;
                if (r < vdim)
                    acc[i] = fmaf(w, ldc<TC>(v, p.v_transposed ? ((int64_t)g * vdim + r) * p.cache.page_tokens + pt
                                                                 : ((int64_t)pt * G + g) * vdim + r), acc[i]);
            }
        }
        __syncthreads();
    }
    float inv = sig ? 1.0f : 1.0f / l_run;
    if (p.gate_col >= 0 && !p.gate_elem) inv *= 1.0f / (1.0f + expf(-p.proj[(int64_t)t * p.ld + p.gate_col + h]));
#pragma unroll
    for (int i = 0; i < GA_MAXV; i++) {
        const int r = tid + i * 256;
        if (r < vdim) {
            float o = acc[i] * inv;
            if (p.gate_col >= 0 && p.gate_elem) o *= 1.0f / (1.0f + expf(-p.proj[(int64_t)t * p.ld + p.gate_col + h * vdim + r]));
            ob[r] = o;
        }
    }
    __syncthreads();
    const float* vcs = p.rot_values ? p.vrope_cos + (int64_t)pos * (vdim / 2) : nullptr;
    const float* vsn = p.rot_values ? p.vrope_sin + (int64_t)pos * (vdim / 2) : nullptr;
    const int64_t o0 = (int64_t)t * p.ld_out + p.out_col + (int64_t)h * vdim;
    for (int r = tid; r < vdim; r += 256) {
        const float o = (p.rot_values ? turned(ob, r, vdim, p.rot_layout, vcs, vsn, -1.f) : ob[r]) * p.out_scale;
        p.out[o0 + r] = o;
        if (p.out_bf) p.out_bf[o0 + r] = f2bf(o);
    }
}

int gqa_attention(const GqaAttnP& p, bool cache_f32, int T, hipStream_t st) {
    QIE_REQUIRE(p.vdim <= 256 * GA_MAXV, "gqa attention: vdim %d above %d", p.vdim, 256 * GA_MAXV);
    QIE_REQUIRE(p.mask == 0 || p.mask_size >= 1, "gqa attention: mask size %d", p.mask_size);
    QIE_REQUIRE(p.heads % p.kv_heads == 0, "gqa attention: %d query heads over %d key heads", p.heads, p.kv_heads);
    const size_t shm = (size_t)(p.dim + GA_CHUNK + p.vdim) * 4;
    QIE_REQUIRE(shm <= 48 * 1024, "gqa attention: head size above the kernel's staging");
    if (cache_f32)
        hipLaunchKernelGGL(gqa_attention_kernel<float>, dim3(p.heads, T), dim3(256), shm, st, p);
    else
        hipLaunchKernelGGL(gqa_attention_kernel<uint16_t>, dim3(p.heads, T), dim3(256), shm, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ attention on the matrix cores
// S^T = K Q^T per 32 keys (two 16 x 16 tiles, K rows as A fragments straight from the cache, the
// queries as bf16 B fragments in registers), masks, bias and the running maximum / sum per
// column in fp32 (a column's 32 scores live in 4 lanes), then O^T += V^T P^T with the softmax
// weights as the B fragment in the order the score tiles left them: k-slot e of lane group g is
// key 4g + e (e < 4) or 16 + 4g + e - 4, which the transposed V rows serve with two 8-byte loads.
// No LDS, no barrier: waves of a workgroup are independent (they share key heads through the L1).
typedef __bf16 gbf16x8_t __attribute__((ext_vector_type(8)));
typedef float gf32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float xg_max(float v) {   // over the 4 lanes n, n + 16, n + 32, n + 48
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    return fmaxf(v, __shfl_xor(v, 32, 64));
}
__device__ __forceinline__ float xg_sum(float v) {
    v += __shfl_xor(v, 16, 64);
    return v + __shfl_xor(v, 32, 64);
}

// heads of one key head that a group of n_tok tokens packs into its 16 columns
__host__ __device__ __forceinline__ int heads_per_token(int n_tok, int H, int G) {
    const int hpk = H / G;
    return (hpk <= 16 && n_tok * hpk <= 16) ? hpk : 1;
}

// One column's finished value sums o[v] (v = v0 .. v0 + 3 of every 16-tile) -> out: turned back by
// the column's position when asked, scaled, stored with the bf16 image.
template <int DV>
__device__ __forceinline__ void gqa_store(const GqaAttnP& a, const gf32x4_t* acc, float inv, int row, int hh, int qpos, int g) {
    const int vdim = 16 * DV;
    const int64_t o0 = (int64_t)row * a.ld_out + a.out_col + (int64_t)hh * vdim;
    const float* cs = a.rot_values ? a.vrope_cos + (int64_t)qpos * (vdim / 2) : nullptr;
    const float* sn = a.rot_values ? a.vrope_sin + (int64_t)qpos * (vdim / 2) : nullptr;
    // the gates of all of the column's coordinates first: a load placed between the stores below would wait for
    // them (the two arrays may overlap as far as the compiler knows)
    const bool gated = a.gate_col >= 0 && a.gate_elem;
    float gf[DV][4];
    if (gated) {
        const float* gp = a.proj + (int64_t)row * a.ld + a.gate_col + hh * vdim + 4 * g;
#pragma unroll
        for (int dv = 0; dv < DV; dv++)
#pragma unroll
            for (int j = 0; j < 4; j++) gf[dv][j] = gp[16 * dv + j];
#pragma unroll
        for (int dv = 0; dv < DV; dv++)
#pragma unroll
            for (int j = 0; j < 4; j++) gf[dv][j] = 1.0f / (1.0f + __expf(-gf[dv][j]));
    }
#pragma unroll
    for (int dv = 0; dv < DV; dv++) {
        float o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = acc[dv][j] * inv;
        const int v0 = 16 * dv + 4 * g;
        if (a.rot_values) {
            if (a.rot_layout == 1) {   // (v0, v0 + 1), (v0 + 2, v0 + 3): turned back = the angle negated
#pragma unroll
                for (int j = 0; j < 4; j += 2) {
                    const float c = cs[(v0 + j) >> 1], s = sn[(v0 + j) >> 1];
                    const float u = o[j], w = o[j + 1];
                    o[j] = u * c + w * s;
                    o[j + 1] = w * c - u * s;
                }
            } else {                   // v with v + vdim / 2: the partner sits DV / 2 tiles away in this lane
                const bool low = dv < DV / 2;
                const int dp = low ? dv + DV / 2 : dv - DV / 2;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int pi = (low ? v0 : v0 - vdim / 2) + j;
                    const float c = cs[pi], s = sn[pi];
                    const float mine = acc[dv][j] * inv, other = acc[dp][j] * inv;
                    o[j] = low ? mine * c + other * s : mine * c - other * s;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float y = o[j] * a.out_scale;
            if (gated) y *= gf[dv][j];
            a.out[o0 + v0 + j] = y;
            if (a.out_bf) a.out_bf[o0 + v0 + j] = f2bf(y);
        }
    }
}

// What a column's value sums are multiplied by: 1 / (sum of its softmax weights), or 1 for sigmoid
// weights; times the head's sigmoid gate when the mixer has one.
// (m: the maximum the weights were taken against; a sink joins the sum as exp(sink_h - m))
__device__ __forceinline__ float gqa_out_factor(const GqaAttnP& a, float l, float m, int row, int hh) {
    if (a.sink) l += __expf(a.sink[hh] - m);
    float f = a.pb ? 1.0f : 1.0f / l;
    if (a.gate_col >= 0 && !a.gate_elem) f *= 1.0f / (1.0f + __expf(-a.proj[(int64_t)row * a.ld + a.gate_col + hh]));
    return f;
}

// SHARE: the four waves of a workgroup are four heads of one key head (heads / kv_heads a
// multiple of 4, one head per wave whatever the group's size): every 32-key K tile and V^T tile
// is brought to LDS once per workgroup (next tile in registers meanwhile) and each wave takes
// its fragments from there - a quarter of the cache traffic of four waves loading for themselves.
template <int DK, int DV, bool SHARE>
__global__ __launch_bounds__(256) void gqa_attn_mfma_kernel(GqaAttnMfmaP P) {
    const GqaAttnP& a = P.a;
    constexpr int dim = 32 * DK, vdim = 16 * DV;
    constexpr int KROW = dim + 8, VROW = 32 + 8;   // LDS rows padded by 16 bytes
    __shared__ __align__(16) uint16_t lk[SHARE ? 32 * KROW : 8];
    __shared__ __align__(16) uint16_t lv[SHARE ? vdim * VROW : 8];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 4, n = lane & 15;
    const int4 grp = P.groups[blockIdx.x];
    const int n_tok = grp.y, slot = grp.z, pos0 = grp.w;
    const int H = a.heads, G = a.kv_heads;
    const int hpt = SHARE ? 1 : heads_per_token(n_tok, H, G);
    const int tile = blockIdx.y * 4 + wave, h0 = SHARE ? min(tile, H - 1) : tile * hpt;
    const bool active = SHARE ? tile < H : true;
    if (!SHARE && h0 >= H) return;
    const int tI = n / hpt, hh = h0 + n % hpt;
    const bool valid = active && tI < n_tok;
    const int tC = valid ? tI : n_tok - 1;
    const int qpos = pos0 + tC, row = grp.x + tC;
    const int kvh = h0 / (H / G);
    // queries: B fragments (column n, k-slots 8g .. 8g + 7 of every 32 coordinates)
    gbf16x8_t qf[DK];
    {
        const float* qr = a.proj + (int64_t)row * a.ld + a.q_col + hh * dim + 8 * g;
#pragma unroll
        for (int ks = 0; ks < DK; ks++) {
            float x[8];
#pragma unroll
            for (int i = 0; i < 8; i++) x[i] = qr[32 * ks + i];
            const uint4 u = make_uint4(pack2(x[0], x[1]), pack2(x[2], x[3]), pack2(x[4], x[5]), pack2(x[6], x[7]));
            qf[ks] = __builtin_bit_cast(gbf16x8_t, u);
        }
    }
    const int lo_q = first_visible(a.mask, a.mask_size, qpos);
    const int kmin = first_visible(a.mask, a.mask_size, pos0), kmax = pos0 + n_tok - 1;
    const int b0 = kmin >> 5, nb = (kmax >> 5) - b0 + 1;
    const int S = P.S, z = blockIdx.z;
    const int bs = b0 + (int)((int64_t)nb * z / S), be = b0 + (int)((int64_t)nb * (z + 1) / S);
    const float b1 = a.r1 ? a.r1[hh] : 0.f, b2 = a.r1 ? a.r2[hh] : 0.f;
    const float slope = a.slopes ? a.slopes[hh] : 0.f;
    const bool sig = a.pb != nullptr;   // sigmoid weights: final as computed, no running maximum or sum
    const float pbh = sig ? a.pb[hh] : 0.f;
    const int PT = a.cache.page_tokens;
    const uint16_t* pool = (const uint16_t*)a.cache.pool;
    const int32_t* tab = a.cache.table + (int64_t)slot * a.cache.max_pages;
    float m_run = sig ? 0.f : -1e30f, l_run = sig ? 1.f : 0.f;
    gf32x4_t acc[DV];
#pragma unroll
    for (int dv = 0; dv < DV; dv++) acc[dv] = gf32x4_t{0.f, 0.f, 0.f, 0.f};
    // K fragments of a 32-key block: two 16-key tiles x DK steps of 32 coordinates; the next
    // block's are loaded while this block is scored, the block's V fragments before its softmax
    uint4 kf[2][DK], kn[2][DK];
    auto load_k = [&](int kb, uint4 (&dst)[2][DK]) {
        const int key0 = kb << 5;
        const int64_t pb = (int64_t)tab[key0 / PT] * a.cache.page_stride;
        const int tok0 = key0 % PT;
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
            const uint16_t* kr = pool + pb + a.k_off + ((int64_t)(tok0 + 16 * tt + n) * G + kvh) * dim + 8 * g;
#pragma unroll
            for (int ks = 0; ks < DK; ks++) dst[tt][ks] = *reinterpret_cast<const uint4*>(kr + 32 * ks);
        }
    };
    // SHARE: a thread's 16-byte pieces of the workgroup's tiles (K: 32 keys x dim, V^T: vdim x 32 keys)
    constexpr int NKP = (32 * dim / 8 + 255) / 256, NVP = (vdim * 4 + 255) / 256;
    uint4 gk[NKP], gv[NVP];
    auto fetch_tiles = [&](int kb) {
        const int key0 = kb << 5;
        const int64_t pb = (int64_t)tab[key0 / PT] * a.cache.page_stride;
        const int tok0 = key0 % PT;
#pragma unroll
        for (int k = 0; k < NKP; k++) {
            const int c = (int)threadIdx.x + 256 * k, key = c / (dim / 8), part = c % (dim / 8);
            if (c < 32 * dim / 8) gk[k] = *reinterpret_cast<const uint4*>(pool + pb + a.k_off + ((int64_t)(tok0 + key) * G + kvh) * dim + part * 8);
        }
#pragma unroll
        for (int k = 0; k < NVP; k++) {
            const int c = (int)threadIdx.x + 256 * k, r = c >> 2, part = c & 3;
            if (c < vdim * 4) gv[k] = *reinterpret_cast<const uint4*>(pool + pb + a.v_off + ((int64_t)kvh * vdim + r) * PT + tok0 + part * 8);
        }
    };
    auto store_tiles = [&]() {
#pragma unroll
        for (int k = 0; k < NKP; k++) {
            const int c = (int)threadIdx.x + 256 * k, key = c / (dim / 8), part = c % (dim / 8);
            if (c < 32 * dim / 8) *reinterpret_cast<uint4*>(lk + key * KROW + part * 8) = gk[k];
        }
#pragma unroll
        for (int k = 0; k < NVP; k++) {
            const int c = (int)threadIdx.x + 256 * k, r = c >> 2, part = c & 3;
            if (c < vdim * 4) *reinterpret_cast<uint4*>(lv + r * VROW + part * 8) = gv[k];
        }
    };
    if (bs < be) {
        if (SHARE) fetch_tiles(bs);
        else load_k(bs, kf);
    }
    for (int kb = bs; kb < be; kb++) {
        const int key0 = kb << 5;
        const int64_t pb = (int64_t)tab[key0 / PT] * a.cache.page_stride;
        const int tok0 = key0 % PT;
        uint2 vf[DV][2];
        if (SHARE) {
            __syncthreads();   // the previous tiles have been read
            store_tiles();
            __syncthreads();
            if (kb + 1 < be) fetch_tiles(kb + 1);
#pragma unroll
            for (int tt = 0; tt < 2; tt++)
#pragma unroll
                for (int ks = 0; ks < DK; ks++) kf[tt][ks] = *reinterpret_cast<const uint4*>(lk + (16 * tt + n) * KROW + 32 * ks + 8 * g);
#pragma unroll
            for (int dv = 0; dv < DV; dv++) {
                vf[dv][0] = *reinterpret_cast<const uint2*>(lv + (16 * dv + n) * VROW + 4 * g);
                vf[dv][1] = *reinterpret_cast<const uint2*>(lv + (16 * dv + n) * VROW + 16 + 4 * g);
            }
        } else {
            const uint16_t* vr = pool + pb + a.v_off + ((int64_t)kvh * vdim + n) * PT + tok0 + 4 * g;
#pragma unroll
            for (int dv = 0; dv < DV; dv++) {
                vf[dv][0] = *reinterpret_cast<const uint2*>(vr + (int64_t)16 * dv * PT);
                vf[dv][1] = *reinterpret_cast<const uint2*>(vr + (int64_t)16 * dv * PT + 16);
            }
            if (kb + 1 < be) load_k(kb + 1, kn);
        }
        gf32x4_t sacc[2];
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
            sacc[tt] = gf32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < DK; ks++)
                sacc[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(gbf16x8_t, kf[tt][ks]), qf[ks], sacc[tt], 0, 0, 0);
        }
        float s[8];
        bool vis[8];
        float bm = -1e30f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int kj = key0 + 16 * (e >> 2) + 4 * g + (e & 3);
            vis[e] = valid && kj >= lo_q && kj <= qpos;
            float x = sacc[e >> 2][e & 3] * a.scale;
            if (a.r1) x -= b1 * __logf(1.0f + b2 * (float)max(qpos - kj, 0));
            x -= slope * (float)max(qpos - kj, 0);
            s[e] = vis[e] ? x : -1e30f;
            bm = fmaxf(bm, s[e]);
        }
        float alpha = 1.0f, pv[8];
        if (sig) {
#pragma unroll
            for (int e = 0; e < 8; e++) pv[e] = vis[e] ? 1.0f / (1.0f + __expf(-(s[e] + pbh))) : 0.f;
        } else {
            bm = xg_max(bm);
            const float m_new = fmaxf(m_run, bm);
            alpha = __expf(m_run - m_new);
            float ls = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                pv[e] = vis[e] ? __expf(s[e] - m_new) : 0.f;
                ls += pv[e];
            }
            ls = xg_sum(ls);
            l_run = l_run * alpha + ls;
            m_run = m_new;
        }
        const uint4 pu = make_uint4(pack2(pv[0], pv[1]), pack2(pv[2], pv[3]), pack2(pv[4], pv[5]), pack2(pv[6], pv[7]));
        const gbf16x8_t pf = __builtin_bit_cast(gbf16x8_t, pu);
#pragma unroll
        for (int dv = 0; dv < DV; dv++) {
            const uint4 vu = make_uint4(vf[dv][0].x, vf[dv][0].y, vf[dv][1].x, vf[dv][1].y);
            if (!sig) {
#pragma unroll
                for (int j = 0; j < 4; j++) acc[dv][j] *= alpha;
            }
            acc[dv] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(gbf16x8_t, vu), pf, acc[dv], 0, 0, 0);
        }
        if (!SHARE) {
#pragma unroll
            for (int tt = 0; tt < 2; tt++)
#pragma unroll
                for (int ks = 0; ks < DK; ks++) kf[tt][ks] = kn[tt][ks];
        }
    }
    if (!active) return;
    if (S == 1) {
        if (valid) gqa_store<DV>(a, acc, gqa_out_factor(a, l_run, m_run, row, hh), row, hh, qpos, g);
        return;
    }
    const int64_t unit = ((int64_t)blockIdx.x * (gridDim.y * 4) + tile) * S + z;
    float* po = P.part_o + (unit * 16 + n) * vdim + 4 * g;
#pragma unroll
    for (int dv = 0; dv < DV; dv++) *reinterpret_cast<float4*>(po + 16 * dv) = make_float4(acc[dv][0], acc[dv][1], acc[dv][2], acc[dv][3]);
    if (g == 0) {
        P.part_ml[(unit * 16 + n) * 2] = m_run;
        P.part_ml[(unit * 16 + n) * 2 + 1] = l_run;
    }
}

// Second pass of a split launch: one wave per (group, tile), the same lane layout as the first.
template <int DV>
__global__ __launch_bounds__(256) void gqa_attn_combine_kernel(GqaAttnMfmaP P, int tiles) {
    const GqaAttnP& a = P.a;
    constexpr int vdim = 16 * DV;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 4, n = lane & 15;
    const int4 grp = P.groups[blockIdx.x];
    const int n_tok = grp.y, pos0 = grp.w;
    const int hpt = P.pack ? heads_per_token(n_tok, a.heads, a.kv_heads) : 1;
    const int tile = blockIdx.y * 4 + wave, h0 = tile * hpt;
    if (h0 >= a.heads) return;
    const int tI = n / hpt, hh = h0 + n % hpt;
    if (tI >= n_tok) return;
    const int64_t u0 = ((int64_t)blockIdx.x * tiles + tile) * P.S;
    const float* ml = P.part_ml + (u0 * 16 + n) * 2;          // part z at ml + 32 z
    float M = -1e30f;
    for (int z = 0; z < P.S; z++) M = fmaxf(M, ml[32 * z]);
    float L = 0.f;
    gf32x4_t acc[DV];
#pragma unroll
    for (int dv = 0; dv < DV; dv++) acc[dv] = gf32x4_t{0.f, 0.f, 0.f, 0.f};
    // several parts a turn (a turn is one trip to memory), every load of the turn issued before its first use; a
    // part that saw no key of the column has l = 0 and zero sums
    constexpr int PT = DV <= 8 ? 4 : 2;
    for (int z0 = 0; z0 < P.S; z0 += PT) {
        float w[PT];
        float4 o[PT][DV];
#pragma unroll
        for (int k = 0; k < PT; k++) {
            const int zk = min(z0 + k, P.S - 1);
            const float l = ml[32 * zk + 1];
            w[k] = (z0 + k >= P.S || l == 0.f) ? 0.f : __expf(ml[32 * zk] - M);
            L += l * w[k];
            const float* pk = P.part_o + ((u0 + zk) * 16 + n) * vdim + 4 * g;
#pragma unroll
            for (int dv = 0; dv < DV; dv++) o[k][dv] = *reinterpret_cast<const float4*>(pk + 16 * dv);
        }
#pragma unroll
        for (int k = 0; k < PT; k++)
#pragma unroll
            for (int dv = 0; dv < DV; dv++) {
                acc[dv][0] += o[k][dv].x * w[k];
                acc[dv][1] += o[k][dv].y * w[k];
                acc[dv][2] += o[k][dv].z * w[k];
                acc[dv][3] += o[k][dv].w * w[k];
            }
    }
    gqa_store<DV>(a, acc, gqa_out_factor(a, L, M, grp.x + tI, hh), grp.x + tI, hh, pos0 + tI, g);
}

bool gqa_attention_mfma_fits(int dim, int vdim, int page_tokens) {
    auto one_of = [](int x, int unit) { return x == unit || x == 2 * unit || x == 4 * unit || x == 8 * unit; };
    return one_of(dim, 32) && one_of(vdim, 32) && page_tokens % 32 == 0;
}

template <int DK, int DV>
static void gqa_mfma_launch2(const GqaAttnMfmaP& p, dim3 grid, hipStream_t st) {
    if (p.pack)
        hipLaunchKernelGGL((gqa_attn_mfma_kernel<DK, DV, false>), grid, dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL((gqa_attn_mfma_kernel<DK, DV, true>), grid, dim3(256), 0, st, p);
    if (p.S > 1) hipLaunchKernelGGL(gqa_attn_combine_kernel<DV>, dim3(grid.x, grid.y, 1), dim3(256), 0, st, p, (int)grid.y * 4);
}
template <int DK>
static int gqa_mfma_launch(const GqaAttnMfmaP& p, dim3 grid, hipStream_t st) {
    switch (p.a.vdim / 32) {
        case 1: gqa_mfma_launch2<DK, 2>(p, grid, st); break;
        case 2: gqa_mfma_launch2<DK, 4>(p, grid, st); break;
        case 4: gqa_mfma_launch2<DK, 8>(p, grid, st); break;
        default: gqa_mfma_launch2<DK, 16>(p, grid, st); break;
    }
    QIE_LAUNCH_CHECK();
    return 0;
}

int gqa_attention_mfma(const GqaAttnMfmaP& p, hipStream_t st) {
    const GqaAttnP& a = p.a;
    QIE_REQUIRE(gqa_attention_mfma_fits(a.dim, a.vdim, a.cache.page_tokens) && a.v_transposed,
                "gqa attention: sizes %d / %d, pages of %d tokens do not fit the matrix-core form", a.dim, a.vdim, a.cache.page_tokens);
    QIE_REQUIRE(p.n_groups > 0 && p.S >= 1 && (p.S == 1 || (p.part_o && p.part_ml)), "gqa attention: bad launch");
    QIE_REQUIRE(a.heads % a.kv_heads == 0, "gqa attention: %d query heads over %d key heads", a.heads, a.kv_heads);
    QIE_REQUIRE(p.pack == ((a.heads / a.kv_heads) % 4 != 0), "gqa attention: packing goes with head ratios that are no multiple of 4");
    dim3 grid((unsigned)p.n_groups, (unsigned)((a.heads + 3) / 4), (unsigned)p.S);
    switch (a.dim / 32) {
        case 1: return gqa_mfma_launch<1>(p, grid, st);
        case 2: return gqa_mfma_launch<2>(p, grid, st);
        case 4: return gqa_mfma_launch<4>(p, grid, st);
        default: return gqa_mfma_launch<8>(p, grid, st);
    }
}

// ------------------------------------------------------------------ gated linear recurrence
// One block per (head, entry, 64 value columns).  A thread owns one column of SR state rows in
// registers; blockDim / 64 thread groups split the dim rows.  The entry's rows go through in
// tiles: the tile's q, f (activations applied, fp32) and v are staged in LDS, every token then
// costs SR multiply-adds per thread with no synchronisation; the groups' partial outputs meet in
// LDS once a tile.  Rows beyond dim are padded with f = 1, q = 0 (their state stays 0).  mode 1
// writes (not adds) its share to out: the caller passes a buffer of its own and sums later.
constexpr int SR = 32;

// TT rows per tile.  The next tile's projection values are loaded into registers while the
// current tile is computed (a block is one to sixteen waves on a CU of its own: nothing else
// would hide the loads), activated and stored to LDS once the tile is done.
template <int TT, int MAXT>
__global__ __launch_bounds__(MAXT) void gated_scan_kernel(GatedScanP p, int dimP) {
    extern __shared__ __align__(16) float sm[];
    const int NG = blockDim.x >> 6;
    float* qs = sm;                       // [TT][dimP]
    float* fs = qs + TT * dimP;           // [TT][dimP]
    float* vs = fs + TT * dimP;           // [TT][64]
    float* op = vs + TT * 64;             // [TT][NG][64]
    const int h = blockIdx.x, c0 = blockIdx.z * 64, tid = threadIdx.x, lane = tid & 63, grp = tid >> 6;
    const int4 en = p.entries[blockIdx.y];
    const int dim = p.dim, vdim = p.vdim, c = c0 + lane, d0 = grp * SR;
    const bool cok = c < vdim;
    float* stp = p.state + (int64_t)en.z * p.slot_stride + p.state_off + (int64_t)h * dim * vdim;
    float S[SR];
#pragma unroll
    for (int r = 0; r < SR; r++) {
        const int d = d0 + r;
        S[r] = ((en.w > 0 || p.mode == 1) && d < dim && cok) ? stp[(int64_t)d * vdim + c] : 0.f;
    }
    const int64_t HV = (int64_t)p.heads * vdim;
    float run = 1.0f;   // thread d < dimP: product of the entry's gates of row d so far
    // a thread stages elements i = tid + k * blockDim of the tile's [TT][dimP] q / f and [TT][64] v
    constexpr int EQ = TT / 2, EV = TT;   // dimP = 32 NG, blockDim = 64 NG
    float rq[EQ], rf[EQ], rv[EV];
    auto fetch = [&](int t0) {
        const int nt = min(TT, en.y - t0);
#pragma unroll
        for (int k = 0; k < EQ; k++) {
            const int i = tid + k * blockDim.x, tt = i / dimP, d = i % dimP;
            rq[k] = 0.f;
            rf[k] = 0.f;
            if (tt < nt && d < dim) {
                const float* row = p.proj + (int64_t)(en.x + t0 + tt) * p.ld;
                rq[k] = row[p.q_col + h * dim + d];
                rf[k] = row[p.f_col + h * dim + d];
            }
        }
#pragma unroll
        for (int k = 0; k < EV; k++) {
            const int i = tid + k * blockDim.x, tt = i >> 6, cc = c0 + (i & 63);
            rv[k] = (i < TT * 64 && tt < nt && cc < vdim) ? p.proj[(int64_t)(en.x + t0 + tt) * p.ld + p.v_col + h * vdim + cc] : 0.f;
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int k = 0; k < EQ; k++) {
            const int i = tid + k * blockDim.x, d = i % dimP;
            float qv = 0.f, fv = 1.f;
            if (d < dim) {
                qv = rq[k] / (1.0f + expf(-rq[k]));
                const float zf = rf[k] + p.f_bias[h * dim + d];
                const float l = p.lower[h * dim + d];
                fv = l + (1.0f - l) * (1.0f / (1.0f + expf(-zf)));
            }
            qs[i] = qv;
            fs[i] = fv;
        }
#pragma unroll
        for (int k = 0; k < EV; k++) {
            const int i = tid + k * blockDim.x;
            if (i < TT * 64) vs[i] = rv[k];
        }
    };
    fetch(0);
    for (int t0 = 0; t0 < en.y; t0 += TT) {
        const int nt = min(TT, en.y - t0);
        __syncthreads();   // the previous tile's readers are done
        stage();
        __syncthreads();
        if (t0 + TT < en.y) fetch(t0 + TT);
        if (p.mode == 1 || p.decay) {
            if (tid < dimP)
                for (int tt = 0; tt < nt; tt++) {
                    run *= fs[tt * dimP + tid];
                    if (p.mode == 1) qs[tt * dimP + tid] *= run;
                }
            __syncthreads();
        }
        if (p.mode == 0) {
            for (int tt = 0; tt < nt; tt++) {
                const float v = vs[tt * 64 + lane];
                const float4* ft = reinterpret_cast<const float4*>(fs + tt * dimP + d0);
                const float4* qt = reinterpret_cast<const float4*>(qs + tt * dimP + d0);
                float o = 0.f;
#pragma unroll
                for (int r4 = 0; r4 < SR / 4; r4++) {
                    const float4 f4 = ft[r4], q4 = qt[r4];
                    const float f[4] = {f4.x, f4.y, f4.z, f4.w}, q[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        S[4 * r4 + j] = fmaf(f[j], S[4 * r4 + j], (1.0f - f[j]) * v);
                        o = fmaf(S[4 * r4 + j], q[j], o);
                    }
                }
                op[(tt * NG + grp) * 64 + lane] = o;
            }
        } else {
            for (int tt = 0; tt < nt; tt++) {
                const float4* qt = reinterpret_cast<const float4*>(qs + tt * dimP + d0);
                float o = 0.f;
#pragma unroll
                for (int r4 = 0; r4 < SR / 4; r4++) {
                    const float4 q4 = qt[r4];
                    o = fmaf(S[4 * r4], q4.x, o);
                    o = fmaf(S[4 * r4 + 1], q4.y, o);
                    o = fmaf(S[4 * r4 + 2], q4.z, o);
                    o = fmaf(S[4 * r4 + 3], q4.w, o);
                }
                op[(tt * NG + grp) * 64 + lane] = o;
            }
        }
        __syncthreads();
        for (int i = tid; i < nt * 64; i += blockDim.x) {
            const int tt = i >> 6, cl = i & 63;
            float o = 0.f;
            for (int gI = 0; gI < NG; gI++) o += op[(tt * NG + gI) * 64 + cl];
            if (c0 + cl < vdim) p.out[(int64_t)(en.x + t0 + tt) * HV + (int64_t)h * vdim + c0 + cl] = o;
        }
    }
    if (p.mode == 1) return;
#pragma unroll
    for (int r = 0; r < SR; r++) {
        const int d = d0 + r;
        if (d < dim && cok) stp[(int64_t)d * vdim + c] = S[r];
    }
    if (p.decay && blockIdx.z == 0 && tid < dim) p.decay[((int64_t)blockIdx.y * p.heads + h) * dim + tid] = run;
}

int gated_scan(const GatedScanP& p, hipStream_t st) {
    QIE_REQUIRE(p.n_entries > 0 && p.heads > 0 && p.dim > 0 && p.vdim > 0, "gated scan: bad sizes");
    const int NG = (p.dim + SR - 1) / SR;
    QIE_REQUIRE(NG <= 16, "gated scan: dim %d above %d", p.dim, 16 * SR);
    const int dimP = NG * SR;
    const int per_tok = (2 * dimP + 64 + NG * 64) * 4;
    dim3 grid((unsigned)p.heads, (unsigned)p.n_entries, (unsigned)((p.vdim + 63) / 64));
    // up to 4 row groups: 256 threads at most, and the register budget that goes with them
    if (NG <= 4)
        hipLaunchKernelGGL((gated_scan_kernel<16, 256>), grid, dim3(64 * NG), (size_t)16 * per_tok, st, p, dimP);
    else if (16 * per_tok <= 60 * 1024)
        hipLaunchKernelGGL((gated_scan_kernel<16, 1024>), grid, dim3(64 * NG), (size_t)16 * per_tok, st, p, dimP);
    else
        hipLaunchKernelGGL((gated_scan_kernel<4, 1024>), grid, dim3(64 * NG), (size_t)4 * per_tok, st, p, dimP);
    QIE_LAUNCH_CHECK();
    return 0;
}

// s_in[c] = the state that enters piece c; one thread per state element walks its entry's pieces.
__global__ __launch_bounds__(256) void gated_carry_kernel(GatedCarryP p) {
    const int64_t n = (int64_t)p.heads * p.dim * p.vdim;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int4 sp = p.spans[blockIdx.y];
    const int64_t hd = i / p.vdim;   // (head, row) of the element: its gate product
    float* stp = p.state + (int64_t)sp.z * p.slot_stride + p.state_off + i;
    float S = sp.w > 0 ? *stp : 0.f;
    for (int c = sp.x; c < sp.x + sp.y; c++) {
        p.s_in[(int64_t)c * n + i] = S;
        S = fmaf(p.decay[(int64_t)c * p.heads * p.dim + hd], S, p.s_loc[(int64_t)c * n + i]);
    }
    *stp = S;
}
int gated_carry(const GatedCarryP& p, hipStream_t st) {
    QIE_REQUIRE(p.n_spans > 0 && p.s_loc && p.decay && p.s_in && p.state, "gated carry: bad arguments");
    const int64_t n = (int64_t)p.heads * p.dim * p.vdim;
    hipLaunchKernelGGL(gated_carry_kernel, dim3((unsigned)((n + 255) / 256), (unsigned)p.n_spans), dim3(256), 0, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ minGRU
// One thread per (entry, channel); the entry's rows go through in order, the loads of a few rows
// ahead are independent of the recurrence, so they overlap it.
__global__ __launch_bounds__(256) void mingru_scan_kernel(MinGruScanP p) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= p.n) return;
    const int4 en = p.entries[blockIdx.y];
    float S = 0.f;
    if (p.init && (!p.init_if_pos || en.w > 0)) S = p.init[(int64_t)en.z * p.init_stride + p.init_off + c];
    const float zb = p.z_b[c], xb = p.x_b[c];
    float run = 1.0f;
    const float* row = p.proj + (int64_t)en.x * p.ld;
    constexpr int U = 4;
    for (int t0 = 0; t0 < en.y; t0 += U) {
        float rz[U], rx[U], rg[U];
#pragma unroll
        for (int k = 0; k < U; k++) {
            const bool on = t0 + k < en.y;
            const float* r = row + (int64_t)(on ? t0 + k : t0) * p.ld;
            rz[k] = r[p.z_col + c];
            rx[k] = r[p.x_col + c];
            rg[k] = p.out ? r[p.g_col + c] : 0.f;
        }
#pragma unroll
        for (int k = 0; k < U; k++) {
            if (t0 + k >= en.y) break;
            const float z = 1.0f / (1.0f + expf(-(rz[k] + zb)));
            const float u = rx[k] + xb;
            const float cand = u >= 0.f ? u + 0.5f : 1.0f / (1.0f + expf(-u));
            S = (1.0f - z) * S + z * cand;
            run *= 1.0f - z;
            if (p.out) {
                const float o = S * (rg[k] / (1.0f + expf(-rg[k])));
                const int64_t oi = (int64_t)(en.x + t0 + k) * p.ld_out + c;
                p.out[oi] = o;
                if (p.out_bf) p.out_bf[oi] = f2bf(o);
            }
        }
    }
    if (p.end) p.end[(int64_t)en.z * p.end_stride + p.end_off + c] = S;
    if (p.decay) p.decay[(int64_t)en.z * p.end_stride + p.end_off + c] = run;
}
int mingru_scan(const MinGruScanP& p, hipStream_t st) {
    QIE_REQUIRE(p.n_entries > 0 && p.n > 0 && p.proj && p.entries && p.z_b && p.x_b && (p.out || p.end), "mingru scan: bad arguments");
    hipLaunchKernelGGL(mingru_scan_kernel, dim3((unsigned)((p.n + 255) / 256), (unsigned)p.n_entries), dim3(256), 0, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

__global__ __launch_bounds__(256) void mingru_carry_kernel(MinGruCarryP p) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= p.n) return;
    const int4 sp = p.spans[blockIdx.y];
    float* stp = p.state + (int64_t)sp.z * p.slot_stride + p.state_off + c;
    float S = sp.w > 0 ? *stp : 0.f;
    for (int k = sp.x; k < sp.x + sp.y; k++) {
        p.s_in[(int64_t)k * p.n + c] = S;
        S = fmaf(p.decay[(int64_t)k * p.n + c], S, p.s_loc[(int64_t)k * p.n + c]);
    }
    *stp = S;
}
int mingru_carry(const MinGruCarryP& p, hipStream_t st) {
    QIE_REQUIRE(p.n_spans > 0 && p.n > 0 && p.s_loc && p.decay && p.s_in && p.state, "mingru carry: bad arguments");
    hipLaunchKernelGGL(mingru_carry_kernel, dim3((unsigned)((p.n + 255) / 256), (unsigned)p.n_spans), dim3(256), 0, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ per-head norm
__global__ __launch_bounds__(256) void head_norm_rows_kernel(const float* o, const float* o2, const float* w, float eps, float scale,
                                                             int heads, int vdim, float* out, uint16_t* out_bf, int64_t ld_out,
                                                             int out_col, const float* gate) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int h = blockIdx.y * 4 + wave; h < heads; h += 4 * gridDim.y) {
        const float* x = o + (t * heads + h) * vdim;
        const float* x2 = o2 ? o2 + (t * heads + h) * vdim : nullptr;
        float ss = 0.f;
        for (int i = lane; i < vdim; i += 64) {
            const float a = x2 ? x[i] + x2[i] : x[i];
            ss += a * a;
        }
        ss = wsum(ss);
        const float inv = scale / sqrtf(ss / (float)vdim + eps);
        const int64_t o0 = t * ld_out + out_col + (int64_t)h * vdim;
        for (int i = lane; i < vdim; i += 64) {
            float y = (x2 ? x[i] + x2[i] : x[i]) * inv * w[i];
            if (gate) y *= 1.0f / (1.0f + expf(-gate[(t * heads + h) * vdim + i]));
            out[o0 + i] = y;
            if (out_bf) out_bf[o0 + i] = f2bf(y);
        }
    }
}
int head_norm_rows(const float* o, const float* o2, const float* w, float eps, float scale, int heads, int vdim, int T, float* out,
                   uint16_t* out_bf, int64_t ld_out, int out_col, hipStream_t st, const float* gate) {
    const int ny = T <= 64 ? std::min(8, (heads + 3) / 4) : 1;   // few rows: a row's heads over several blocks
    hipLaunchKernelGGL(head_norm_rows_kernel, dim3(T, ny), dim3(256), 0, st, o, o2, w, eps, scale, heads, vdim, out, out_bf, ld_out,
                       out_col, gate);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ residual add + next norm
__global__ __launch_bounds__(256) void add_norm_kernel(float* x, const float* xin, const float* v, const float* wb, const float* add,
                                                       const float* wn, float* h, uint16_t* h_bf, int W, float eps, float w_one, int copies,
                                                       int64_t plane) {
    __shared__ float red[4];
    const int64_t r0 = (int64_t)blockIdx.x * W;
    float inv_v = 0.f;
    if (v && wb) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < W; i += 256) {
            const float a = v[r0 + i];
            ss += a * a;
        }
        ss = bsum256(ss, red);
        inv_v = 1.0f / sqrtf(ss / (float)W + eps);
    }
    float sx = 0.f;
    for (int i = threadIdx.x; i < W; i += 256) {
        float a = xin[r0 + i];
        if (v) a += wb ? v[r0 + i] * inv_v * (w_one + wb[i]) : v[r0 + i];
        if (add) a += add[r0 + i];
        if (v || add || xin != x) x[r0 + i] = a;
        sx += a * a;
    }
    if (!wn) return;
    sx = bsum256(sx, red);
    const float inv_x = 1.0f / sqrtf(sx / (float)W + eps);
    for (int i = threadIdx.x; i < W; i += 256) {
        const float o = x[r0 + i] * inv_x * (w_one + wn[i]);   // the thread's own store above
        h[r0 + i] = o;
        for (int k = 1; k < copies; k++) h[k * plane + r0 + i] = o;
        if (h_bf) h_bf[r0 + i] = f2bf(o);
    }
}
int add_norm(float* x, const float* xin, const float* v, const float* wb, const float* add, const float* wn, float* h, uint16_t* h_bf,
             int T, int W, float eps, hipStream_t st, float w_one, int copies, int64_t plane) {
    QIE_REQUIRE(x && xin && (!wn || h), "add_norm: bad arguments");
    hipLaunchKernelGGL(add_norm_kernel, dim3(T), dim3(256), 0, st, x, xin, v, wb, add, wn, h, h_bf, W, eps, w_one, copies, plane);
    QIE_LAUNCH_CHECK();
    return 0;
}

}  // namespace lay
}  // namespace qie
