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
//
// Long entries run in pieces side by side.  A column s of S moves through a row as s <- A_t s + beta k v_c
// with A_t = (I - beta k k^T) diag(g), the same A_t for every column, so over a piece s_end = M s_in + s_loc with
// M = the product of the piece's A_t and s_loc the end state from zero.  A piece scanned from zero with dim extra
// columns that start as the unit vectors and see v = 0 yields s_loc, M (those columns' end states) and, as those
// columns' outputs, w_t = M_t^T q_t, M_t the product up to row t.  lay::delta_carry walks an entry's pieces
// (s_in of the next piece = M s_in + s_loc; the slot's state = what leaves the last), lay::delta_apply adds the
// incoming state's share s_in^T w_t to every row's output: no second scan.  Same sums as row by row up to fp32
// rounding.
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

// gridDim.y blocks per row (several when the step has few rows); a wave per (q or k) head, then the gates.
__global__ __launch_bounds__(256) void delta_prep_kernel(DeltaPrepP p) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, y = blockIdx.y, ny = gridDim.y;
    float* qk = p.qkv + t * p.ld_qkv;
    const float qs = 1.0f / sqrtf((float)p.dim);
    for (int hh = y * 4 + wave; hh < 2 * p.G; hh += 4 * ny) {
        float* x = qk + (int64_t)hh * p.dim;   // q heads, then k heads
        float ss = 0.f;
        for (int i = lane; i < p.dim; i += 64) ss += x[i] * x[i];
        ss = wsum64(ss);
        const float inv = (hh < p.G ? qs : 1.0f) / sqrtf(ss + 1e-6f);
        for (int i = lane; i < p.dim; i += 64) x[i] *= inv;
    }
    float* row = p.proj + t * p.ld;
    if (y == 0)
        for (int h = threadIdx.x; h < p.H; h += 256) row[p.b_col + h] = 1.0f / (1.0f + expf(-row[p.b_col + h]));
    float* a = p.a + t * (int64_t)p.H * p.dim;
    for (int i = y * 256 + threadIdx.x; i < p.H * p.dim; i += 256 * ny) {
        const float z = a[i] + p.dt_bias[i];
        const float sp = fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)));
        a[i] = expf(-p.exp_a[i / p.dim] * sp);
    }
}

int delta_prep(const DeltaPrepP& p, int T, hipStream_t st) {
    QIE_REQUIRE(p.qkv && p.proj && p.a && p.dt_bias && p.exp_a && p.H > 0 && p.G > 0 && p.H % p.G == 0 && p.dim > 0,
                "delta_prep: bad arguments");
    const int ny = T <= 64 ? std::min(8, std::max(1, p.H * p.dim / 256)) : 1;
    hipLaunchKernelGGL(delta_prep_kernel, dim3(T, ny), dim3(256), 0, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

constexpr int DS_RP = 32;   // state rows per lane
constexpr int DS_TT = 8;    // rows staged at a time
constexpr int DS_SEG = DS_RP + 4;   // a lane group's 32 staged values, padded by 16 bytes: the LP groups of a column read
                                    // different banks (unpadded they sit 128 bytes apart, the same banks)

template <int LP>
__global__ __launch_bounds__(256) void delta_scan_kernel(DeltaScanP p) {
    extern __shared__ float sm[];
    constexpr int dimP = DS_RP * LP, dimS = DS_SEG * LP, CPB = 256 / LP;
    float* sq = sm;
    float* sk = sm + DS_TT * dimS;
    float* sg = sm + 2 * DS_TT * dimS;
    float* sb = sm + 3 * DS_TT * dimS;
    const int h = blockIdx.x, tid = threadIdx.x, rg = tid % LP, col = blockIdx.z * CPB + tid / LP;
    const int4 en = p.entries[blockIdx.y];   // {first packed row, rows, slot, first position}
    const int dim = p.dim, vdim = p.vdim, G = p.G, H = p.H;
    const int gh = h / (H / G);
    // columns vdim .. vdim + dim - 1 (when p.trans): the unit vectors under v = 0, see the header
    const bool colv = col < vdim + (p.trans ? dim : 0), idc = col >= vdim;
    const int64_t HV = (int64_t)H * vdim, HD = (int64_t)H * dim;
    float* stp = p.state + (int64_t)en.z * p.slot_stride + p.state_off + (int64_t)h * dim * vdim;
    const bool rd = p.read_state == 2 || (p.read_state == 1 && en.w > 0);
    float S[DS_RP];
#pragma unroll
    for (int i = 0; i < DS_RP; i++) {
        const int r = rg * DS_RP + i;
        S[i] = idc ? (r == col - vdim ? 1.f : 0.f) : (rd && colv && r < dim) ? stp[(int64_t)r * vdim + col] : 0.f;
    }
    const int v_col = 2 * G * dim + h * vdim + col;
    for (int t0 = 0; t0 < en.y; t0 += DS_TT) {
        const int nt = min(DS_TT, en.y - t0);
        float vv[DS_TT];
#pragma unroll
        for (int tt = 0; tt < DS_TT; tt++) vv[tt] = (tt < nt && colv && !idc) ? p.qkv[(int64_t)(en.x + t0 + tt) * p.ld_qkv + v_col] : 0.f;
        __syncthreads();   // the previous rows have been read
        for (int i = tid; i < nt * dimP; i += 256) {
            const int tt = i / dimP, r = i % dimP;
            const int64_t row = en.x + t0 + tt;
            const bool in = r < dim;
            const float* qr = p.qkv + row * p.ld_qkv;
            const int d = tt * dimS + (r / DS_RP) * DS_SEG + r % DS_RP;
            sq[d] = in ? qr[gh * dim + r] : 0.f;
            sk[d] = in ? qr[(G + gh) * dim + r] : 0.f;
            sg[d] = in ? p.g[row * HD + (int64_t)h * dim + r] : 1.f;
        }
        if (tid < nt) sb[tid] = p.beta[(int64_t)(en.x + t0 + tid) * p.ld_beta + h];
        __syncthreads();
        for (int tt = 0; tt < nt; tt++) {
            const float* kk = sk + tt * dimS + rg * DS_SEG;
            const float* qq = sq + tt * dimS + rg * DS_SEG;
            const float* gg = sg + tt * dimS + rg * DS_SEG;
            // four partial sums per inner product: the adds of one sum wait for each other
            float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
            for (int i = 0; i < DS_RP; i += 4) {
                const float4 g4 = *reinterpret_cast<const float4*>(gg + i);
                const float4 k4 = *reinterpret_cast<const float4*>(kk + i);
                S[i] *= g4.x; S[i + 1] *= g4.y; S[i + 2] *= g4.z; S[i + 3] *= g4.w;
                d0 = fmaf(k4.x, S[i], d0);
                d1 = fmaf(k4.y, S[i + 1], d1);
                d2 = fmaf(k4.z, S[i + 2], d2);
                d3 = fmaf(k4.w, S[i + 3], d3);
            }
            const float dot = group_sum_lp<LP>((d0 + d1) + (d2 + d3));
            const float u = sb[tt] * (vv[tt] - dot);
            float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
            for (int i = 0; i < DS_RP; i += 4) {
                const float4 k4 = *reinterpret_cast<const float4*>(kk + i);
                const float4 q4 = *reinterpret_cast<const float4*>(qq + i);
                S[i] = fmaf(k4.x, u, S[i]);
                S[i + 1] = fmaf(k4.y, u, S[i + 1]);
                S[i + 2] = fmaf(k4.z, u, S[i + 2]);
                S[i + 3] = fmaf(k4.w, u, S[i + 3]);
                o0 = fmaf(q4.x, S[i], o0);
                o1 = fmaf(q4.y, S[i + 1], o1);
                o2 = fmaf(q4.z, S[i + 2], o2);
                o3 = fmaf(q4.w, S[i + 3], o3);
            }
            const float o = group_sum_lp<LP>((o0 + o1) + (o2 + o3));
            if (rg == 0 && colv) {
                if (!idc)
                    p.out[(int64_t)(en.x + t0 + tt) * HV + (int64_t)h * vdim + col] = o;
                else
                    p.w_out[(int64_t)(en.x + t0 + tt) * HD + (int64_t)h * dim + (col - vdim)] = o;
            }
        }
    }
    if (!colv) return;
    if (idc) {   // column col - vdim of the piece's transition matrix
        float* mt = p.trans + ((int64_t)en.z * H + h) * dim * dim + (col - vdim);
#pragma unroll
        for (int i = 0; i < DS_RP; i++) {
            const int r = rg * DS_RP + i;
            if (r < dim) mt[(int64_t)r * dim] = S[i];
        }
        return;
    }
    if (!p.write_state) return;
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
    QIE_REQUIRE(!p.trans || p.w_out, "delta_scan: the transition matrices go with the rows' transformed queries");
    const int cpb = 256 / LP, ncols = p.vdim + (p.trans ? p.dim : 0);
    const dim3 grid((unsigned)p.H, (unsigned)p.n_entries, (unsigned)((ncols + cpb - 1) / cpb));
    const size_t shm = (size_t)(3 * DS_TT * DS_SEG * LP + DS_TT) * 4;
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

// ------------------------------------------------------------------ pieces: carry and apply
// One block per (entry, head, 8 state columns): the columns live in LDS, thread (r0, c) owns rows r0, r0 + 32, ...
constexpr int DC_COLS = 8;

__global__ __launch_bounds__(256) void delta_carry_kernel(DeltaCarryP p) {
    extern __shared__ float ss[];   // [dim][DC_COLS]
    const int4 sp = p.spans[blockIdx.x];   // {first piece, pieces, slot, first position}
    const int h = blockIdx.y, c = threadIdx.x % DC_COLS, r0 = threadIdx.x / DC_COLS, col = blockIdx.z * DC_COLS + c;
    const int dim = p.dim, vdim = p.vdim, H = p.H;
    const bool colv = col < vdim;
    float* stp = p.state + (int64_t)sp.z * p.slot_stride + p.state_off + (int64_t)h * dim * vdim;
    for (int r = r0; r < dim; r += 32) ss[r * DC_COLS + c] = (sp.w > 0 && colv) ? stp[(int64_t)r * vdim + col] : 0.f;
    __syncthreads();
    const int nr = (dim - r0 + 31) / 32;   // this thread's rows r0, r0 + 32, ... (at most 16)
    for (int k = 0; k < sp.y; k++) {
        const int64_t ph = (int64_t)(sp.x + k) * H + h;
        const float* mt = p.trans + ph * dim * dim;
        float acc[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int r = r0 + 32 * i;
            acc[i] = 0.f;
            if (i < nr && colv) {
                p.s_in[(ph * dim + r) * vdim + col] = ss[r * DC_COLS + c];
                acc[i] = p.s_loc[(ph * dim + r) * vdim + col];
            }
        }
        // rows in groups of four share every read of the state column; four matrix entries per load where dim allows
        for (int i0 = 0; i0 < nr; i0 += 4) {
            float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
            const float* m0 = mt + (int64_t)(r0 + 32 * i0) * dim;
            const float* m1 = m0 + (i0 + 1 < nr ? 32 * dim : 0);
            const float* m2 = m0 + (i0 + 2 < nr ? 64 * dim : 0);
            const float* m3 = m0 + (i0 + 3 < nr ? 96 * dim : 0);
            int j = 0;
            if ((dim & 3) == 0) {
                for (; j < dim; j += 4) {
                    const float4 x0 = *reinterpret_cast<const float4*>(m0 + j), x1 = *reinterpret_cast<const float4*>(m1 + j);
                    const float4 x2 = *reinterpret_cast<const float4*>(m2 + j), x3 = *reinterpret_cast<const float4*>(m3 + j);
                    const float s0 = ss[j * DC_COLS + c], s1 = ss[(j + 1) * DC_COLS + c], s2 = ss[(j + 2) * DC_COLS + c],
                                s3 = ss[(j + 3) * DC_COLS + c];
                    a0 = fmaf(x0.w, s3, fmaf(x0.z, s2, fmaf(x0.y, s1, fmaf(x0.x, s0, a0))));
                    a1 = fmaf(x1.w, s3, fmaf(x1.z, s2, fmaf(x1.y, s1, fmaf(x1.x, s0, a1))));
                    a2 = fmaf(x2.w, s3, fmaf(x2.z, s2, fmaf(x2.y, s1, fmaf(x2.x, s0, a2))));
                    a3 = fmaf(x3.w, s3, fmaf(x3.z, s2, fmaf(x3.y, s1, fmaf(x3.x, s0, a3))));
                }
            }
            for (; j < dim; j++) {
                const float sv = ss[j * DC_COLS + c];
                a0 = fmaf(m0[j], sv, a0);
                a1 = fmaf(m1[j], sv, a1);
                a2 = fmaf(m2[j], sv, a2);
                a3 = fmaf(m3[j], sv, a3);
            }
#pragma unroll
            for (int i = 0; i < 16; i += 4)
                if (i == i0) {
                    acc[i] += a0;
                    acc[i + 1] += a1;
                    acc[i + 2] += a2;
                    acc[i + 3] += a3;
                }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int r = r0 + 32 * i;
            if (i < nr) ss[r * DC_COLS + c] = acc[i];
        }
        __syncthreads();
    }
    if (!p.write_state || !colv) return;
    for (int r = r0; r < dim; r += 32) stp[(int64_t)r * vdim + col] = ss[r * DC_COLS + c];
}

int delta_carry(const DeltaCarryP& p, hipStream_t st) {
    QIE_REQUIRE(p.spans && p.n_spans > 0 && p.s_loc && p.trans && p.s_in && p.state && p.dim > 0 && p.dim <= 512 && p.vdim > 0,
                "delta_carry: bad arguments");
    const dim3 grid((unsigned)p.n_spans, (unsigned)p.H, (unsigned)((p.vdim + DC_COLS - 1) / DC_COLS));
    hipLaunchKernelGGL(delta_carry_kernel, grid, dim3(256), (size_t)p.dim * DC_COLS * 4, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

// out[t, h, col] += sum_j s_in[piece][h][j][col] w[t, h, j]: one block per (piece, head, 64 columns), j in tiles of 64
// through LDS; thread (rq, col) owns rows rq, rq + 4, ... of the piece (at most 64).
__global__ __launch_bounds__(256) void delta_apply_kernel(DeltaApplyP p) {
    __shared__ float sw[64 * 64];   // [row][j]
    __shared__ float st[64 * 64];   // [j][col]
    const int4 en = p.chunks[blockIdx.x];   // {first packed row, rows, piece index, 0}
    const int h = blockIdx.y, lc = threadIdx.x & 63, rq = threadIdx.x >> 6, col = blockIdx.z * 64 + lc;
    const int dim = p.dim, vdim = p.vdim, H = p.H;
    const float* sin = p.s_in + ((int64_t)en.z * H + h) * dim * vdim;
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
    for (int j0 = 0; j0 < dim; j0 += 64) {
        __syncthreads();
        for (int i = threadIdx.x; i < 64 * 64; i += 256) {
            const int a = i >> 6, bq = i & 63;   // w: row a, j bq;  state: j a, column bq
            sw[i] = (a < en.y && j0 + bq < dim) ? p.w[(int64_t)(en.x + a) * H * dim + (int64_t)h * dim + j0 + bq] : 0.f;
            st[i] = (j0 + a < dim && blockIdx.z * 64 + bq < vdim) ? sin[(int64_t)(j0 + a) * vdim + blockIdx.z * 64 + bq] : 0.f;
        }
        __syncthreads();
        for (int jj = 0; jj < 64; jj++) {
            const float sv = st[jj * 64 + lc];
#pragma unroll
            for (int i = 0; i < 16; i++) acc[i] = fmaf(sw[(rq + 4 * i) * 64 + jj], sv, acc[i]);
        }
    }
    if (col >= vdim) return;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int a = rq + 4 * i;
        if (a < en.y) p.out[(int64_t)(en.x + a) * H * vdim + (int64_t)h * vdim + col] += acc[i];
    }
}

int delta_apply(const DeltaApplyP& p, hipStream_t st) {
    QIE_REQUIRE(p.chunks && p.n_chunks > 0 && p.s_in && p.w && p.out && p.max_rows <= 64, "delta_apply: bad arguments (pieces of at most 64 rows)");
    const dim3 grid((unsigned)p.n_chunks, (unsigned)p.H, (unsigned)((p.vdim + 63) / 64));
    hipLaunchKernelGGL(delta_apply_kernel, grid, dim3(256), 0, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

}  // namespace lay
}  // namespace qie
