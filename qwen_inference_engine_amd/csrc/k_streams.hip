// k_streams.hip — residual-stream mechanisms of the layered engine tier (k_layered.hpp):
//
//   lay::stream_step        several residual rows per token mixed by learned coefficients
//                           (hyper-connections): the update after a sublayer fused with the
//                           read-out and the norm that feed the next sublayer
//   lay::causal_conv        causal convolution over time per channel on the packed rows of a ragged
//                           step; rows before an entry's first come from the slot's state
//   lay::causal_conv_state  advances that state by the entry's rows
//   lay::rms_rows           RMS norm of a column range of every row
//
// fp32 throughout.  A row's result depends on its own slot's rows and state only.
#include "k_layered.hpp"

namespace qie {
namespace lay {

namespace {
__device__ __forceinline__ float wsum64(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float bsum(float v, float* red) {
    v = wsum64(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}
}  // namespace

// ------------------------------------------------------------------ hyper-connections
// One block per row.  A thread owns coordinates w = tid, tid + 256, ... of all N rows of its token:
// new rows from the old ones, the read-out u, u kept in LDS for the norm's second pass.  NT: the number of rows
// at compile time (1 .. 8), or 0 for any number up to kMaxStreams.
constexpr int kMaxStreams = 32;

template <int NT>
__global__ __launch_bounds__(256) void stream_step_kernel(StreamStepP p, int stage) {
    extern __shared__ float su[];   // [W]
    __shared__ float red[4];
    constexpr int NA = NT ? NT : kMaxStreams;
    const int N = NT ? NT : p.n;
    const int64_t r0 = (int64_t)blockIdx.x * p.W;
    // the coefficient tables: the same addresses for every lane (scalar loads, in flight beside the rows' loads);
    // an unknown number of rows keeps them in LDS instead
    __shared__ float cms[NT ? 1 : NA * NA + 2 * NA];
    float cmr[NT ? NT * NT + 2 * NT : 1];
    if (NT) {
#pragma unroll
        for (int i = 0; i < NT * NT; i++) cmr[i] = p.y ? p.mix[i] : 0.f;
#pragma unroll
        for (int i = 0; i < NT; i++) {
            cmr[NT * NT + i] = p.y ? p.out[i] : 0.f;
            cmr[NT * NT + NT + i] = p.in ? p.in[i] : 0.f;
        }
    } else {
        for (int i = threadIdx.x; i < N * N; i += 256) cms[i] = p.y ? p.mix[i] : 0.f;
        if (threadIdx.x < N) {
            cms[N * N + threadIdx.x] = p.y ? p.out[threadIdx.x] : 0.f;
            cms[N * N + N + threadIdx.x] = p.in ? p.in[threadIdx.x] : 0.f;
        }
        __syncthreads();
    }
    const float* cm = NT ? cmr : cms;
    float ss = 0.f;
    for (int w = threadIdx.x; w < p.W; w += 256) {
        float x[NA];
#pragma unroll
        for (int s = 0; s < N; s++) x[s] = p.X[s * p.plane + r0 + w];
        if (p.y) {
            const float y = p.y[r0 + w];
            float nx[NA];
#pragma unroll
            for (int t = 0; t < N; t++) {
                float a = cm[N * N + t] * y;
#pragma unroll
                for (int s = 0; s < N; s++) a = fmaf(cm[s * N + t], x[s], a);
                nx[t] = a;
            }
#pragma unroll
            for (int t = 0; t < N; t++) {
                x[t] = nx[t];
                p.X[t * p.plane + r0 + w] = nx[t];
            }
        }
        if (p.sum) {
            float a = 0.f;
#pragma unroll
            for (int s = 0; s < N; s++) a += x[s];
            p.sum[r0 + w] = a;
        }
        if (p.in) {
            float u = 0.f;
#pragma unroll
            for (int s = 0; s < N; s++) u = fmaf(cm[N * N + N + s], x[s], u);
            if (stage) su[w] = u;
            ss += u * u;
        }
    }
    if (!p.in) return;
    ss = bsum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)p.W + p.eps);
    for (int w = threadIdx.x; w < p.W; w += 256) {
        float u = 0.f;
        if (stage) {
            u = su[w];   // the thread's own LDS store above
        } else {         // rows wider than the staging: the read-out again from the thread's own stores, same order
#pragma unroll
            for (int s = 0; s < N; s++) u = fmaf(cm[N * N + N + s], p.X[s * p.plane + r0 + w], u);
        }
        const float o = u * inv * (p.w_one + p.wn[w]);
        p.h[r0 + w] = o;
        if (p.h_bf) p.h_bf[r0 + w] = f2bf(o);
    }
}

int stream_step(const StreamStepP& p, hipStream_t st) {
    QIE_REQUIRE(p.n >= 1 && p.n <= kMaxStreams && p.X && p.T > 0 && p.W > 0, "stream_step: %d streams (at most %d)", p.n, kMaxStreams);
    QIE_REQUIRE(!p.y || (p.mix && p.out), "stream_step: an update needs its coefficients");
    QIE_REQUIRE(!p.in || (p.wn && p.h), "stream_step: a read-out needs its norm weight and a destination");
    const int stage = (size_t)p.W * 4 <= 48 * 1024 ? 1 : 0;
    const size_t shm = stage ? (size_t)p.W * 4 : 0;
#define QIE_SS(N) hipLaunchKernelGGL(stream_step_kernel<N>, dim3(p.T), dim3(256), shm, st, p, stage)
    switch (p.n) {
        case 1: QIE_SS(1); break;
        case 2: QIE_SS(2); break;
        case 3: QIE_SS(3); break;
        case 4: QIE_SS(4); break;
        case 5: QIE_SS(5); break;
        case 6: QIE_SS(6); break;
        case 7: QIE_SS(7); break;
        case 8: QIE_SS(8); break;
        default: QIE_SS(0); break;
    }
#undef QIE_SS
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ causal convolution over time
// One thread per (row, channel).  Tap j reaches back taps - 1 - j rows: inside the row's entry it
// reads the step's rows, before the entry's first row the slot's state (the last taps - 1 inputs
// before the entry, oldest first), before the sequence's start zero.
__global__ __launch_bounds__(256) void causal_conv_kernel(CausalConvP p, int T) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)T * p.C) return;
    const int t = (int)(i / p.C), c = (int)(i % p.C);
    const int slot = p.row_slot[t], pos = p.row_pos[t], k = p.row_k[t];
    const float* w = p.w + (int64_t)c * p.taps;
    const float* sb = p.state + (int64_t)slot * p.slot_stride + p.state_off;
    const float cur = p.in[(int64_t)t * p.ld_in + p.col + c];
    float a = 0.f;
    for (int j = 0; j < p.taps; j++) {
        const int back = p.taps - 1 - j;
        float x;
        if (back == 0)
            x = cur;
        else if (back <= k)
            x = p.in[(int64_t)(t - back) * p.ld_in + p.col + c];
        else if (pos - back >= 0)
            x = sb[(int64_t)(k - back + p.taps - 1) * p.C + c];
        else
            x = 0.f;
        a = fmaf(w[j], x, a);
    }
    if (p.residual) a += cur;
    if (p.silu) a = a / (1.0f + expf(-a));
    const int64_t o = (int64_t)t * p.ld_out + c;
    p.out[o] = a;
    if (p.out_bf) p.out_bf[o] = f2bf(a);
}

// One thread per (entry, channel): state row i becomes the input at position p1 - (taps - 1) + i,
// p1 the position after the entry's last row.  Ascending i reads old rows i + count > i before any
// of them is written.
__global__ __launch_bounds__(256) void causal_conv_state_kernel(CausalConvP p) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= p.C) return;
    const int4 en = p.entries[blockIdx.y];   // {first packed row, rows, slot, first position}
    float* sb = p.state + (int64_t)en.z * p.slot_stride + p.state_off;
    const int n = p.taps - 1;
    for (int i = 0; i < n; i++) {
        const int q = en.y - n + i;          // row of the entry that lands in state row i (negative: before it)
        float x;
        if (q >= 0)
            x = p.in[(int64_t)(en.x + q) * p.ld_in + p.col + c];
        else if (en.w + q >= 0)
            x = sb[(int64_t)(i + en.y) * p.C + c];
        else
            x = 0.f;
        sb[(int64_t)i * p.C + c] = x;
    }
}

// Steps of few rows: one thread per (entry, channel) does both - the entry's rows in order, then the state - in one
// launch (the thread reads the old state for its rows before it writes the new one).
__global__ __launch_bounds__(256) void causal_conv_fused_kernel(CausalConvP p) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= p.C) return;
    const int4 en = p.entries[blockIdx.y];   // {first packed row, rows, slot, first position}
    float* sb = p.state + (int64_t)en.z * p.slot_stride + p.state_off;
    const float* w = p.w + (int64_t)c * p.taps;
    for (int k = 0; k < en.y; k++) {
        const int t = en.x + k, pos = en.w + k;
        const float cur = p.in[(int64_t)t * p.ld_in + p.col + c];
        float a = 0.f;
        for (int j = 0; j < p.taps; j++) {
            const int back = p.taps - 1 - j;
            float x;
            if (back == 0)
                x = cur;
            else if (back <= k)
                x = p.in[(int64_t)(t - back) * p.ld_in + p.col + c];
            else if (pos - back >= 0)
                x = sb[(int64_t)(k - back + p.taps - 1) * p.C + c];
            else
                x = 0.f;
            a = fmaf(w[j], x, a);
        }
        if (p.residual) a += cur;
        if (p.silu) a = a / (1.0f + expf(-a));
        const int64_t o = (int64_t)t * p.ld_out + c;
        p.out[o] = a;
        if (p.out_bf) p.out_bf[o] = f2bf(a);
    }
    const int n = p.taps - 1;
    for (int i = 0; i < n; i++) {
        const int q = en.y - n + i;
        float x;
        if (q >= 0)
            x = p.in[(int64_t)(en.x + q) * p.ld_in + p.col + c];
        else if (en.w + q >= 0)
            x = sb[(int64_t)(i + en.y) * p.C + c];
        else
            x = 0.f;
        sb[(int64_t)i * p.C + c] = x;
    }
}

static int conv_check(const CausalConvP& p) {
    QIE_REQUIRE(p.in && p.w && p.C > 0 && p.taps >= 1 && p.taps <= 64, "causal_conv: %d channels, %d taps", p.C, p.taps);
    QIE_REQUIRE(p.taps == 1 || p.state, "causal_conv: the state is missing");
    return 0;
}
int causal_conv(const CausalConvP& p, int T, hipStream_t st) {
    QIE_TRY(conv_check(p));
    QIE_REQUIRE(p.out && p.row_slot && p.row_pos && p.row_k, "causal_conv: bad arguments");
    const int64_t n = (int64_t)T * p.C;
    hipLaunchKernelGGL(causal_conv_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, p, T);
    QIE_LAUNCH_CHECK();
    return 0;
}
int causal_conv_advance(const CausalConvP& p, int T, hipStream_t st) {
    QIE_TRY(conv_check(p));
    QIE_REQUIRE(p.out && p.entries && p.n_entries > 0, "causal_conv_advance: bad arguments");
    if (T > kConvFusedRows || p.out == p.in) {
        QIE_TRY(causal_conv(p, T, st));
        return causal_conv_state(p, st);
    }
    hipLaunchKernelGGL(causal_conv_fused_kernel, dim3((unsigned)((p.C + 255) / 256), (unsigned)p.n_entries), dim3(256), 0, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}
int causal_conv_state(const CausalConvP& p, hipStream_t st) {
    QIE_TRY(conv_check(p));
    if (p.taps == 1) return 0;
    QIE_REQUIRE(p.entries && p.n_entries > 0, "causal_conv_state: bad arguments");
    hipLaunchKernelGGL(causal_conv_state_kernel, dim3((unsigned)((p.C + 255) / 256), (unsigned)p.n_entries), dim3(256), 0, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ norm of a column range
// out[t, c] = in[t, col + c] / sqrt(mean_c in^2 + eps) * (w_one + w[c]), c < n
__global__ __launch_bounds__(256) void rms_rows_kernel(const float* in, int64_t ld_in, int col, int n, const float* w, float w_one,
                                                       float eps, float* out, int64_t ld_out, uint16_t* out_bf) {
    __shared__ float red[4];
    const float* x = in + (int64_t)blockIdx.x * ld_in + col;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) ss += x[i] * x[i];
    ss = bsum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += 256) {
        const float o = x[i] * inv * (w_one + w[i]);
        out[(int64_t)blockIdx.x * ld_out + i] = o;
        if (out_bf) out_bf[(int64_t)blockIdx.x * ld_out + i] = f2bf(o);
    }
}
int rms_rows(const float* in, int64_t ld_in, int col, int n, const float* w, float w_one, float eps, float* out, int64_t ld_out,
             uint16_t* out_bf, int T, hipStream_t st) {
    QIE_REQUIRE(in && w && out && n > 0, "rms_rows: bad arguments");
    hipLaunchKernelGGL(rms_rows_kernel, dim3(T), dim3(256), 0, st, in, ld_in, col, n, w, w_one, eps, out, ld_out, out_bf);
    QIE_LAUNCH_CHECK();
    return 0;
}

}  // namespace lay
}  // namespace qie
