// layered_ssm.hip — blocks of layers whose two sublayers read one norm, with a token shift in front of the mixer (kernels/layered.h): the norm with the shift, the
// input of a pass over a looped range, the front (causal convolution, step sizes) and the end (skip, gate, group norm) of a state-space mixer whose recurrence is
// retention's token-gated form, rotated queries and keys on their way into the pages, the mixes of a time-mixing recurrence.  Norms, angles, step sizes, decays and scores are f32 in both operand types.  wave64, gfx950.
#include <hip/hip_runtime.h>
#include <math.h>
#include <algorithm>
#include "../common.h"
#include "layered.h"

namespace nvr { namespace kl {

namespace {

typedef uint16_t bf16_t;
__device__ __forceinline__ float ld_f(const float *p, int64_t i) { return p[i]; }
__device__ __forceinline__ float ld_f(const bf16_t *p, int64_t i) { return __uint_as_float((uint32_t)p[i] << 16); }
__device__ __forceinline__ void st_f(float *p, int64_t i, float v) { p[i] = v; }
__device__ __forceinline__ void st_f(bf16_t *p, int64_t i, float v) {       // round to nearest even
    uint32_t u = __float_as_uint(v);
    if ((u & 0x7fffffffu) > 0x7f800000u) { p[i] = (bf16_t)((u >> 16) | 0x40); return; }
    u += 0x7fffu + ((u >> 16) & 1u);
    p[i] = (bf16_t)(u >> 16);
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
// sums of two numbers over the 256 threads of a workgroup; red: 8 floats of LDS; every thread gets both
__device__ __forceinline__ void block_sum2(float &u, float &v, float *red) {
    u = wave_sum(u); v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) { red[threadIdx.x >> 6] = u; red[4 + (threadIdx.x >> 6)] = v; }
    __syncthreads();
    u = (red[0] + red[1]) + (red[2] + red[3]); v = (red[4] + red[5]) + (red[6] + red[7]);
}
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

int launched(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return nvr::fail(NVR_ERR_HIP, "%s launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

// ------------------------------------------------------------------------------------------------ norm + token shift
// One workgroup per row: the row's norm and, where the row before it belongs to the same chunk, that row's norm too (the same arithmetic as that row's own
// workgroup: a cut changes nothing); the first row of a chunk reads the slot's history instead.
template <class OT>
__global__ __launch_bounds__(256) void norm_shift_kernel(const float *__restrict__ x, Batch b, int W, float eps, const float *__restrict__ w, const float *__restrict__ shift,
                                                         OT *__restrict__ out_h, OT *__restrict__ out_m, float *__restrict__ hist, int64_t slots) {
    __shared__ float red[8];
    const int t = blockIdx.x, sq = b.row_seq[t];
    const int i = t - b.cu[sq], n = b.cu[sq + 1] - b.cu[sq], st = b.start[sq];
    const float *xr = x + (int64_t)t * W, *xp = xr - W;
    const bool inside = i > 0;
    float s1 = 0.f, s0 = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) { const float v = xr[c]; s1 += v * v; if (inside) { const float u = xp[c]; s0 += u * u; } }
    block_sum2(s1, s0, red);
    const float f1 = 1.0f / sqrtf(s1 / (float)W + eps), f0 = 1.0f / sqrtf(s0 / (float)W + eps);
    const float *hp = (!inside && st > 0) ? hist + ((int64_t)b.par[sq] * slots + b.slot[sq]) * W : nullptr;
    float *hn = i == n - 1 ? hist + ((int64_t)(b.par[sq] ^ 1) * slots + b.slot[sq]) * W : nullptr;
    for (int c = threadIdx.x; c < W; c += 256) {
        const float h = xr[c] * f1 * w[c];
        const float before = inside ? xp[c] * f0 * w[c] : (hp ? hp[c] : 0.f);
        if (out_h) st_f(out_h, (int64_t)t * W + c, h);
        st_f(out_m, (int64_t)t * W + c, h + (before - h) * shift[c]);
        if (hn) hn[c] = h;
    }
}

template <class OT>
__global__ __launch_bounds__(256) void pair_rows_kernel(const float *__restrict__ x, const float *__restrict__ x0, int64_t T, int W, OT *__restrict__ out) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= T * 2 * W) return;
    const int64_t t = idx / (2 * W); const int c = (int)(idx - t * 2 * W);
    st_f(out, idx, c < W ? x[t * W + c] : x0[t * W + c - W]);
}

// ------------------------------------------------------------------------------------------------ state-space mixer: convolution, step sizes
// One workgroup per row.  The input of the convolution d rows back is a row of this step, a row of the slot's history or zero; the chunk's last row also writes the
// slot's new history (the chunk's last taps - 1 inputs, or older ones moved up where the chunk is shorter).
template <class OT>
__global__ __launch_bounds__(256) void conv_gates_kernel(ConvGateArgs a, Batch b) {
    const int t = blockIdx.x, sq = b.row_seq[t];
    const int i = t - b.cu[sq], n = b.cu[sq + 1] - b.cu[sq], st = b.start[sq];
    const int C = a.C, taps = a.taps, back = taps - 1;
    const OT *pr = (const OT *)a.proj + (int64_t)t * a.ld;
    const float *hp = a.hist + ((int64_t)b.par[sq] * a.slots + b.slot[sq]) * back * C;            // inputs of positions st - back .. st - 1
    // the input of channel c at the chunk's row r (r < 0: before the chunk)
    auto input = [&](int r, int c) -> float {
        if (r >= 0) return ld_f((const OT *)a.proj + (int64_t)(t - i + r) * a.ld, a.ccol + c);
        if (st + r < 0) return 0.f;
        return hp[(int64_t)(back + r) * C + c];
    };
    for (int c = threadIdx.x; c < C; c += 256) {
        float acc = a.bias ? a.bias[c] : 0.f;
        for (int j = 0; j < taps; ++j) acc += a.w[(int64_t)c * taps + j] * input(i - back + j, c);
        st_f((OT *)a.out, (int64_t)t * a.ldo + c, silu_f(acc));
    }
    if (threadIdx.x < a.H) {
        const int h = threadIdx.x;
        const float dt = softplus_f(ld_f(pr, a.dcol + h) + a.dt_bias[h]);
        a.tok_gate[((int64_t)t * a.H + h) * 2] = expf(-expf(a.a_log[h]) * dt);
        a.tok_gate[((int64_t)t * a.H + h) * 2 + 1] = dt;
    }
    if (i == n - 1 && back > 0) {
        float *hn = a.hist + ((int64_t)(b.par[sq] ^ 1) * a.slots + b.slot[sq]) * back * C;
        for (int idx = threadIdx.x; idx < back * C; idx += 256) { const int j = idx / C, c = idx - j * C; hn[idx] = input(n - back + j, c); }
    }
}

// ------------------------------------------------------------------------------------------------ state-space mixer: skip, gate, group norm
// One workgroup per row, a wave per group of the norm.
template <class OT>
__global__ __launch_bounds__(256) void state_readout_kernel(StateReadoutArgs a) {
    const int64_t t = blockIdx.x; const int lane = threadIdx.x & 63;
    const int inner = a.H * a.Dv, gs = inner / a.groups;
    const float *o = a.o + t * inner;
    const OT *xs = (const OT *)a.xs + t * a.ldx, *z = (const OT *)a.z + t * a.ldz;
    for (int g = threadIdx.x >> 6; g < a.groups; g += 4) {
        float ss = 0.f;
        for (int c = g * gs + lane; c < (g + 1) * gs; c += 64) { const float y = (o[c] + a.skip[c / a.Dv] * ld_f(xs, c)) * silu_f(ld_f(z, c)); ss += y * y; }
        ss = wave_sum(ss);
        const float f = 1.0f / sqrtf(ss / (float)gs + a.eps);
        for (int c = g * gs + lane; c < (g + 1) * gs; c += 64) {
            const float y = (o[c] + a.skip[c / a.Dv] * ld_f(xs, c)) * silu_f(ld_f(z, c));
            st_f((OT *)a.out, t * a.ldo + c, y * f * a.w[c]);
        }
    }
}

// ------------------------------------------------------------------------------------------------ rotated queries and keys, K / V rows into the pages
template <class CT>
__global__ __launch_bounds__(256) void rope_store_kernel(RopeStoreArgs a, Batch b) {
    const int t = blockIdx.x, sq = b.row_seq[t];
    const int p = b.start[sq] + (t - b.cu[sq]);
    const int blk = b.block_tables[(int64_t)sq * b.max_blocks + p / b.block_size], jj = p % b.block_size;
    const int64_t row = (int64_t)blk * b.block_size + jj;
    CT *pr = (CT *)a.proj + (int64_t)t * a.ld;
    CT *kc = (CT *)a.kc, *vc = (CT *)a.vc;
    const int D = a.D, half = a.rot / 2;
    // queries: the pairs of the rotated part, in place (a thread reads its pair, then writes it)
    for (int idx = threadIdx.x; idx < a.H * half; idx += 256) {
        const int h = idx / half, i = idx - h * half;
        const float ang = (float)p * a.freq[i], cs = cosf(ang), sn = sinf(ang);
        CT *q = pr + a.qcol + (int64_t)h * D;
        const float u = ld_f(q, i), v = ld_f(q, i + half);
        st_f(q, i, u * cs - v * sn); st_f(q, i + half, v * cs + u * sn);
    }
    // keys: every coordinate goes to the page row, the rotated part turned
    for (int idx = threadIdx.x; idx < a.G * D; idx += 256) {
        const int g = idx / D, d = idx - g * D;
        const CT *k = pr + a.kcol + (int64_t)g * D;
        float v = ld_f(k, d);
        if (d < a.rot) {
            const int i = d < half ? d : d - half;
            const float ang = (float)p * a.freq[i], cs = cosf(ang), sn = sinf(ang);
            v = d < half ? v * cs - ld_f(k, d + half) * sn : v * cs + ld_f(k, d - half) * sn;
        }
        st_f(kc, row * a.G * D + idx, v);
    }
    const int GV = a.G * a.Dv;
    if (!a.v_grouped) { for (int c = threadIdx.x; c < GV; c += 256) vc[row * GV + c] = pr[a.vcol + c]; return; }
    const int64_t grp = ((int64_t)blk * (b.block_size >> 3) + (jj >> 3)) * GV;        // value pages in groups of 8 keys per column
    for (int c = threadIdx.x; c < GV; c += 256) vc[(grp + c) * 8 + (jj & 7)] = pr[a.vcol + c];
}

// ------------------------------------------------------------------------------------------------ mixes of a time-mixing layer
template <class OT>
__global__ __launch_bounds__(256) void shift_mixes_kernel(const OT *__restrict__ m, int64_t ldm, Batch b, int W, int nm, const float *__restrict__ mu, OT *__restrict__ out,
                                                          float *__restrict__ hist, int64_t slots) {
    const int t = blockIdx.x, sq = b.row_seq[t];
    const int i = t - b.cu[sq], n = b.cu[sq + 1] - b.cu[sq], st = b.start[sq];
    const OT *mr = m + (int64_t)t * ldm;
    const float *hp = (i == 0 && st > 0) ? hist + ((int64_t)b.par[sq] * slots + b.slot[sq]) * W : nullptr;
    float *hn = i == n - 1 ? hist + ((int64_t)(b.par[sq] ^ 1) * slots + b.slot[sq]) * W : nullptr;
    OT *orow = out + (int64_t)t * nm * W;
    for (int c = threadIdx.x; c < W; c += 256) {
        const float v = ld_f(mr, c);
        const float before = i > 0 ? ld_f(mr - ldm, c) : (hp ? hp[c] : 0.f);
        for (int k = 0; k < nm; ++k) st_f(orow, (int64_t)k * W + c, v + (before - v) * mu[(int64_t)k * W + c]);
        if (hn) hn[c] = v;
    }
}

template <class OT>
__global__ __launch_bounds__(256) void tanh_rows_kernel(OT *__restrict__ y, int64_t ld, int64_t T, int64_t N) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= T * N) return;
    const int64_t t = idx / N, c = idx - t * N;
    st_f(y, t * ld + c, tanhf(ld_f(y, t * ld + c)));
}

}  // namespace

int norm_shift(const float *x, const Batch &b, int64_t W, float eps, const float *w, const float *shift, void *out_h, void *out_m, float *hist, int64_t slots, bool bf16, hipStream_t s) {
    if (b.T == 0) return 0;
    if (bf16) norm_shift_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(256), 0, s>>>(x, b, (int)W, eps, w, shift, (bf16_t *)out_h, (bf16_t *)out_m, hist, slots);
    else norm_shift_kernel<float><<<dim3((unsigned)b.T), dim3(256), 0, s>>>(x, b, (int)W, eps, w, shift, (float *)out_h, (float *)out_m, hist, slots);
    return launched("norm_shift");
}

int pair_rows(const float *x, const float *x0, int64_t T, int64_t W, void *out, bool bf16, hipStream_t s) {
    if (T == 0) return 0;
    const dim3 grid((unsigned)((T * 2 * W + 255) / 256));
    if (bf16) pair_rows_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(x, x0, T, (int)W, (bf16_t *)out);
    else pair_rows_kernel<float><<<grid, dim3(256), 0, s>>>(x, x0, T, (int)W, (float *)out);
    return launched("pair_rows");
}

int conv_gates(const ConvGateArgs &a, const Batch &b, bool bf16, hipStream_t s) {
    if (b.T == 0) return 0;
    if (a.taps < 1 || a.H > 256 || a.H < 1 || a.C < 1) return nvr::fail(NVR_ERR_INVALID_ARG, "conv_gates: %d taps over %d channels, %d heads (at most 256)", a.taps, a.C, a.H);
    if (bf16) conv_gates_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(256), 0, s>>>(a, b);
    else conv_gates_kernel<float><<<dim3((unsigned)b.T), dim3(256), 0, s>>>(a, b);
    return launched("conv_gates");
}

int state_readout(const StateReadoutArgs &a, bool bf16, hipStream_t s) {
    if (a.T == 0) return 0;
    if (a.groups < 1 || (a.H * a.Dv) % a.groups) return nvr::fail(NVR_ERR_INVALID_ARG, "state_readout: %d numbers in %d groups", a.H * a.Dv, a.groups);
    if (bf16) state_readout_kernel<bf16_t><<<dim3((unsigned)a.T), dim3(256), 0, s>>>(a);
    else state_readout_kernel<float><<<dim3((unsigned)a.T), dim3(256), 0, s>>>(a);
    return launched("state_readout");
}

int rope_store(const RopeStoreArgs &a, const Batch &b, bool bf16, hipStream_t s) {
    if (b.T == 0) return 0;
    if (a.rot % 2 || a.rot > a.D || a.rot < 0) return nvr::fail(NVR_ERR_INVALID_ARG, "rope_store: %d rotated coordinates of %d", a.rot, a.D);
    if (a.v_grouped && b.block_size % 8) return nvr::fail(NVR_ERR_INVALID_ARG, "rope_store: grouped value pages need pages of a multiple of 8 tokens");
    if (bf16) rope_store_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(256), 0, s>>>(a, b);
    else rope_store_kernel<float><<<dim3((unsigned)b.T), dim3(256), 0, s>>>(a, b);
    return launched("rope_store");
}

int shift_mixes(const void *m, int64_t ldm, const Batch &b, int64_t W, int32_t n, const float *mu, void *out, float *hist, int64_t slots, bool bf16, hipStream_t s) {
    if (b.T == 0) return 0;
    if (bf16) shift_mixes_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(256), 0, s>>>((const bf16_t *)m, ldm, b, (int)W, (int)n, mu, (bf16_t *)out, hist, slots);
    else shift_mixes_kernel<float><<<dim3((unsigned)b.T), dim3(256), 0, s>>>((const float *)m, ldm, b, (int)W, (int)n, mu, (float *)out, hist, slots);
    return launched("shift_mixes");
}

int tanh_rows(void *y, int64_t ld, int64_t T, int64_t N, bool bf16, hipStream_t s) {
    if (T * N == 0) return 0;
    const dim3 grid((unsigned)((T * N + 255) / 256));
    if (bf16) tanh_rows_kernel<bf16_t><<<grid, dim3(256), 0, s>>>((bf16_t *)y, ld, T, N);
    else tanh_rows_kernel<float><<<grid, dim3(256), 0, s>>>((float *)y, ld, T, N);
    return launched("tanh_rows");
}

}}  // namespace nvr::kl
