// k_delta.hip — the gated delta rule with channel-wise decay (QIE_MIXER_CHANNEL_DELTA; k_layered.hpp):
//
//   lay::delta_prep   per row: q and k of every key head to unit length (q also times dim^(-1/2)),
//                     beta = sigmoid, decay g = exp(-exp(A_log) softplus(a + dt_bias)) - all fp32
//   lay::delta_scan   per entry and head the state S [dim][vdim] walks the entry's rows in order:
//                     S = diag(g) S; u = beta (v - S^T k); S += k u^T; o = S^T q
//
// The columns of S are independent of each other under this rule (each sees only k, q, g, beta and
// its own v), so a column lives in the registers of LP neighbouring lanes (32 rows each) and the
// two inner products of a row are reduced over those lanes by shuffles; a workgroup holds 256 / LP
// columns of one head.  q, k, g and beta of 8 rows at a time are staged in LDS (every lane of a
// column group reads the same addresses), the next rows' values already in registers.  The state
// is fp32 and lives with the slot; an entry that starts at position 0 starts from zero.
#include "k_layered.hpp"

namespace qie {
namespace lay {

namespace {
__device__ __forceinline__ float wsum64(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
template <int LP> __device__ __forceinline__ float group_sum_lp(float v) {
#pragma unroll
    for (int o = LP / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
}  // namespace

// One block per row; a wave per (q or k) head, then the gates.
__global__ __launch_bounds__(256) void delta_prep_kernel(DeltaPrepP p) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float* qk = p.qkv + t * p.ld_qkv;
    const float qs = 1.0f / sqrtf((float)p.dim);
    for (int hh = wave; hh < 2 * p.G; hh += 4) {
        float* x = qk + (int64_t)hh * p.dim;   // q heads, then k heads
        float ss = 0.f;
        for (int i = lane; i < p.dim; i += 64) ss += x[i] * x[i];
        ss = wsum64(ss);
        const float inv = (hh < p.G ? qs : 1.0f) / sqrtf(ss + 1e-6f);
        for (int i = lane; i < p.dim; i += 64) x[i] *= inv;
    }
    float* row = p.proj + t * p.ld;
    for (int h = threadIdx.x; h < p.H; h += 256) row[p.b_col + h] = 1.0f / (1.0f + expf(-row[p.b_col + h]));
    float* a = p.a + t * (int64_t)p.H * p.dim;
    for (int i = threadIdx.x; i < p.H * p.dim; i += 256) {
        const float z = a[i] + p.dt_bias[i];
        const float sp = fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)));
        a[i] = expf(-p.exp_a[i / p.dim] * sp);
    }
}

int delta_prep(const DeltaPrepP& p, int T, hipStream_t st) {
    QIE_REQUIRE(p.qkv && p.proj && p.a && p.dt_bias && p.exp_a && p.H > 0 && p.G > 0 && p.H % p.G == 0 && p.dim > 0,
                "delta_prep: bad arguments");
    hipLaunchKernelGGL(delta_prep_kernel, dim3(T), dim3(256), 0, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

constexpr int DS_RP = 32;   // state rows per lane
constexpr int DS_TT = 8;    // rows staged at a time

template <int LP>
__global__ __launch_bounds__(256) void delta_scan_kernel(DeltaScanP p) {
    extern __shared__ float sm[];
    constexpr int dimP = DS_RP * LP, CPB = 256 / LP;
    float* sq = sm;
    float* sk = sm + DS_TT * dimP;
    float* sg = sm + 2 * DS_TT * dimP;
    float* sb = sm + 3 * DS_TT * dimP;
    const int h = blockIdx.x, tid = threadIdx.x, rg = tid % LP, col = blockIdx.z * CPB + tid / LP;
    const int4 en = p.entries[blockIdx.y];   // {first packed row, rows, slot, first position}
    const int dim = p.dim, vdim = p.vdim, G = p.G, H = p.H;
    const int gh = h / (H / G);
    const bool colv = col < vdim;
    const int64_t HV = (int64_t)H * vdim, HD = (int64_t)H * dim;
    float* stp = p.state + (int64_t)en.z * p.slot_stride + p.state_off + (int64_t)h * dim * vdim;
    float S[DS_RP];
#pragma unroll
    for (int i = 0; i < DS_RP; i++) {
        const int r = rg * DS_RP + i;
        S[i] = (p.read_state && en.w > 0 && colv && r < dim) ? stp[(int64_t)r * vdim + col] : 0.f;
    }
    const int v_col = 2 * G * dim + h * vdim + col;
    for (int t0 = 0; t0 < en.y; t0 += DS_TT) {
        const int nt = min(DS_TT, en.y - t0);
        float vv[DS_TT];
#pragma unroll
        for (int tt = 0; tt < DS_TT; tt++) vv[tt] = (tt < nt && colv) ? p.qkv[(int64_t)(en.x + t0 + tt) * p.ld_qkv + v_col] : 0.f;
        __syncthreads();   // the previous rows have been read
        for (int i = tid; i < nt * dimP; i += 256) {
            const int tt = i / dimP, r = i % dimP;
            const int64_t row = en.x + t0 + tt;
            const bool in = r < dim;
            const float* qr = p.qkv + row * p.ld_qkv;
            sq[i] = in ? qr[gh * dim + r] : 0.f;
            sk[i] = in ? qr[(G + gh) * dim + r] : 0.f;
            sg[i] = in ? p.g[row * HD + (int64_t)h * dim + r] : 1.f;
        }
        if (tid < nt) sb[tid] = p.beta[(int64_t)(en.x + t0 + tid) * p.ld_beta + h];
        __syncthreads();
        for (int tt = 0; tt < nt; tt++) {
            const float* kk = sk + tt * dimP + rg * DS_RP;
            const float* qq = sq + tt * dimP + rg * DS_RP;
            const float* gg = sg + tt * dimP + rg * DS_RP;
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < DS_RP; i += 4) {
                const float4 g4 = *reinterpret_cast<const float4*>(gg + i);
                const float4 k4 = *reinterpret_cast<const float4*>(kk + i);
                S[i] *= g4.x; S[i + 1] *= g4.y; S[i + 2] *= g4.z; S[i + 3] *= g4.w;
                dot = fmaf(k4.x, S[i], dot);
                dot = fmaf(k4.y, S[i + 1], dot);
                dot = fmaf(k4.z, S[i + 2], dot);
                dot = fmaf(k4.w, S[i + 3], dot);
            }
            dot = group_sum_lp<LP>(dot);
            const float u = sb[tt] * (vv[tt] - dot);
            float o = 0.f;
#pragma unroll
            for (int i = 0; i < DS_RP; i += 4) {
                const float4 k4 = *reinterpret_cast<const float4*>(kk + i);
                const float4 q4 = *reinterpret_cast<const float4*>(qq + i);
                S[i] = fmaf(k4.x, u, S[i]);
                S[i + 1] = fmaf(k4.y, u, S[i + 1]);
                S[i + 2] = fmaf(k4.z, u, S[i + 2]);
                S[i + 3] = fmaf(k4.w, u, S[i + 3]);
                o = fmaf(q4.x, S[i], o);
                o = fmaf(q4.y, S[i + 1], o);
                o = fmaf(q4.z, S[i + 2], o);
                o = fmaf(q4.w, S[i + 3], o);
            }
            o = group_sum_lp<LP>(o);
            if (rg == 0 && colv) p.out[(int64_t)(en.x + t0 + tt) * HV + (int64_t)h * vdim + col] = o;
        }
    }
    if (!colv || !p.write_state) return;
#pragma unroll
    for (int i = 0; i < DS_RP; i++) {
        const int r = rg * DS_RP + i;
        if (r < dim) stp[(int64_t)r * vdim + col] = S[i];
    }
}

int delta_scan(const DeltaScanP& p, hipStream_t st) {
    QIE_REQUIRE(p.qkv && p.beta && p.g && p.entries && p.n_entries > 0 && p.state && p.out, "delta_scan: bad arguments");
    QIE_REQUIRE(p.H > 0 && p.G > 0 && p.H % p.G == 0 && p.dim > 0 && p.dim <= 16 * DS_RP && p.vdim > 0,
                "delta_scan: %d heads over %d key heads of %d / %d (dim at most %d)", p.H, p.G, p.dim, p.vdim, 16 * DS_RP);
    int LP = 1;
    while (LP * DS_RP < p.dim) LP *= 2;
    const int cpb = 256 / LP;
    const dim3 grid((unsigned)p.H, (unsigned)p.n_entries, (unsigned)((p.vdim + cpb - 1) / cpb));
    const size_t shm = (size_t)(3 * DS_TT * DS_RP * LP + DS_TT) * 4;
    switch (LP) {
        case 1: hipLaunchKernelGGL(delta_scan_kernel<1>, grid, dim3(256), shm, st, p); break;
        case 2: hipLaunchKernelGGL(delta_scan_kernel<2>, grid, dim3(256), shm, st, p); break;
        case 4: hipLaunchKernelGGL(delta_scan_kernel<4>, grid, dim3(256), shm, st, p); break;
        case 8: hipLaunchKernelGGL(delta_scan_kernel<8>, grid, dim3(256), shm, st, p); break;
        default: hipLaunchKernelGGL(delta_scan_kernel<16>, grid, dim3(256), shm, st, p); break;
    }
    QIE_LAUNCH_CHECK();
    return 0;
}

}  // namespace lay
}  // namespace qie
