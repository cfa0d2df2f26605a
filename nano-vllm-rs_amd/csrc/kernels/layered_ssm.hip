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
    for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += 256 * gridDim.y) {
        float acc = a.bias ? a.bias[c] : 0.f;
        for (int j = 0; j < taps; ++j) acc += a.w[(int64_t)c * taps + j] * input(i - back + j, c);
        st_f((OT *)a.out, (int64_t)t * a.ldo + c, silu_f(acc));
    }
    if (blockIdx.y == 0 && threadIdx.x < a.H) {
        const int h = threadIdx.x;
        const float dt = softplus_f(ld_f(pr, a.dcol + h) + a.dt_bias[h]);
        a.tok_gate[((int64_t)t * a.H + h) * 2] = expf(-expf(a.a_log[h]) * dt);
        a.tok_gate[((int64_t)t * a.H + h) * 2 + 1] = dt;
    }
    if (i == n - 1 && back > 0) {
        float *hn = a.hist + ((int64_t)(b.par[sq] ^ 1) * a.slots + b.slot[sq]) * back * C;
        for (int idx = blockIdx.y * 256 + threadIdx.x; idx < back * C; idx += 256 * gridDim.y) { const int j = idx / C, c = idx - j * C; hn[idx] = input(n - back + j, c); }
    }
}

// 16-bit rows, 8 channels per thread as 16-byte loads and stores (C, both strides and the first column multiples of 8; 16-byte aligned rows), RB consecutive rows of
// the step per workgroup: a thread keeps its channels' weights and the taps - 1 inputs before the current row in registers, so that every input is read once.  The
// window is filled anew at the block's first row and at a chunk's first row (from the step's rows, the slot's history, or zeros before position 0); behind a chunk's
// last row it holds the slot's new history.
template <int TAPS, int RB>
__global__ __launch_bounds__(256) void conv_gates8_kernel(ConvGateArgs a, Batch b) {
    constexpr int BACK = TAPS - 1;
    const int r0 = blockIdx.x * RB, r1 = min(r0 + RB, b.T), C = a.C;
    const int c0 = (blockIdx.y * 256 + threadIdx.x) * 8;
    if (blockIdx.y == 0)
        for (int idx = threadIdx.x; idx < (r1 - r0) * a.H; idx += 256) {
            const int t = r0 + idx / a.H, h = idx % a.H;
            const float dt = softplus_f(ld_f((const bf16_t *)a.proj + (int64_t)t * a.ld, a.dcol + h) + a.dt_bias[h]);
            a.tok_gate[((int64_t)t * a.H + h) * 2] = expf(-expf(a.a_log[h]) * dt);
            a.tok_gate[((int64_t)t * a.H + h) * 2 + 1] = dt;
        }
    if (c0 >= C) return;
    float wr[8][TAPS], bias[8], win[BACK > 0 ? BACK : 1][8];
#pragma unroll
    for (int y = 0; y < 8; ++y) {
        bias[y] = a.bias ? a.bias[c0 + y] : 0.f;
#pragma unroll
        for (int j = 0; j < TAPS; ++j) wr[y][j] = a.w[(int64_t)(c0 + y) * TAPS + j];
    }
    auto load8 = [&](const bf16_t *p, float (&v)[8]) {
        const uint4 u = *reinterpret_cast<const uint4 *>(p);
        const bf16_t *e = reinterpret_cast<const bf16_t *>(&u);
#pragma unroll
        for (int y = 0; y < 8; ++y) v[y] = ld_f(e, y);
    };
    for (int t = r0; t < r1; ++t) {
        const int sq = b.row_seq[t], i = t - b.cu[sq], n = b.cu[sq + 1] - b.cu[sq], st = b.start[sq];
        const bf16_t *pr = (const bf16_t *)a.proj + (int64_t)t * a.ld + a.ccol + c0;
        if (BACK > 0 && (t == r0 || i == 0)) {
            const float *hp = a.hist + ((int64_t)b.par[sq] * a.slots + b.slot[sq]) * BACK * C;
#pragma unroll
            for (int j = 0; j < BACK; ++j) {
                const int r = i - BACK + j;                 // the chunk's row of this tap (negative: before the chunk)
                if (r >= 0) load8(pr + (int64_t)(j - BACK) * a.ld, win[j]);
                else if (st + r < 0) {
#pragma unroll
                    for (int y = 0; y < 8; ++y) win[j][y] = 0.f;
                } else {
                    const float4 lo = *reinterpret_cast<const float4 *>(hp + (int64_t)(BACK + r) * C + c0), hi = *reinterpret_cast<const float4 *>(hp + (int64_t)(BACK + r) * C + c0 + 4);
                    win[j][0] = lo.x; win[j][1] = lo.y; win[j][2] = lo.z; win[j][3] = lo.w; win[j][4] = hi.x; win[j][5] = hi.y; win[j][6] = hi.z; win[j][7] = hi.w;
                }
            }
        }
        float cur[8];
        load8(pr, cur);
        uint4 o; bf16_t *oe = reinterpret_cast<bf16_t *>(&o);
#pragma unroll
        for (int y = 0; y < 8; ++y) {
            float acc = bias[y];
#pragma unroll
            for (int j = 0; j < BACK; ++j) acc += wr[y][j] * win[j][y];
            acc += wr[y][BACK] * cur[y];
            st_f(oe, y, silu_f(acc));
        }
        *reinterpret_cast<uint4 *>((bf16_t *)a.out + (int64_t)t * a.ldo + c0) = o;
#pragma unroll
        for (int j = 0; j + 1 < BACK; ++j)
#pragma unroll
            for (int y = 0; y < 8; ++y) win[j][y] = win[j + 1][y];
        if (BACK > 0)
#pragma unroll
            for (int y = 0; y < 8; ++y) win[BACK - 1][y] = cur[y];
        if (BACK > 0 && i == n - 1) {
            float *hn = a.hist + ((int64_t)(b.par[sq] ^ 1) * a.slots + b.slot[sq]) * BACK * C;
#pragma unroll
            for (int j = 0; j < BACK; ++j) {
                *reinterpret_cast<float4 *>(hn + (int64_t)j * C + c0) = float4{win[j][0], win[j][1], win[j][2], win[j][3]};
                *reinterpret_cast<float4 *>(hn + (int64_t)j * C + c0 + 4) = float4{win[j][4], win[j][5], win[j][6], win[j][7]};
            }
        }
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

// 16-bit rows, 8 channels per thread as 16-byte loads and stores (W and the stride multiples of 8, 16-byte aligned rows)
__global__ __launch_bounds__(256) void shift_mixes8_kernel(const bf16_t *__restrict__ m, int64_t ldm, Batch b, int W, int nm, const float *__restrict__ mu, bf16_t *__restrict__ out,
                                                           float *__restrict__ hist, int64_t slots) {
    const int w8 = W >> 3;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;       // (row, piece of 8 channels): every thread has its own piece
    if (idx >= (int64_t)b.T * w8) return;
    const int t = (int)(idx / w8), c0 = (int)(idx - (int64_t)t * w8) << 3, sq = b.row_seq[t];
    const int i = t - b.cu[sq], n = b.cu[sq + 1] - b.cu[sq], st = b.start[sq];
    const bf16_t *mr = m + (int64_t)t * ldm;
    const float *hp = (i == 0 && st > 0) ? hist + ((int64_t)b.par[sq] * slots + b.slot[sq]) * W : nullptr;
    float *hn = i == n - 1 ? hist + ((int64_t)(b.par[sq] ^ 1) * slots + b.slot[sq]) * W : nullptr;
    bf16_t *orow = out + (int64_t)t * nm * W;
    {
        float v[8], before[8];
        const uint4 u = *reinterpret_cast<const uint4 *>(mr + c0);
        const bf16_t *e = reinterpret_cast<const bf16_t *>(&u);
#pragma unroll
        for (int y = 0; y < 8; ++y) v[y] = ld_f(e, y);
        if (i > 0) {
            const uint4 p = *reinterpret_cast<const uint4 *>(mr - ldm + c0);
            const bf16_t *pe = reinterpret_cast<const bf16_t *>(&p);
#pragma unroll
            for (int y = 0; y < 8; ++y) before[y] = ld_f(pe, y);
        } else {
#pragma unroll
            for (int y = 0; y < 8; ++y) before[y] = 0.f;
            if (hp) {
                const float4 h0 = *reinterpret_cast<const float4 *>(hp + c0), h1 = *reinterpret_cast<const float4 *>(hp + c0 + 4);
                before[0] = h0.x; before[1] = h0.y; before[2] = h0.z; before[3] = h0.w; before[4] = h1.x; before[5] = h1.y; before[6] = h1.z; before[7] = h1.w;
            }
        }
        for (int k = 0; k < nm; ++k) {
            uint4 o; bf16_t *oe = reinterpret_cast<bf16_t *>(&o);
            const float4 m0 = *reinterpret_cast<const float4 *>(mu + (int64_t)k * W + c0), m1 = *reinterpret_cast<const float4 *>(mu + (int64_t)k * W + c0 + 4);
            const float mk[8] = {m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w};
#pragma unroll
            for (int y = 0; y < 8; ++y) st_f(oe, y, v[y] + (before[y] - v[y]) * mk[y]);
            *reinterpret_cast<uint4 *>(orow + (int64_t)k * W + c0) = o;
        }
        if (hn) {
            *reinterpret_cast<float4 *>(hn + c0) = float4{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<float4 *>(hn + c0 + 4) = float4{v[4], v[5], v[6], v[7]};
        }
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
    if (bf16 && a.taps <= 4 && a.C % 8 == 0 && a.ld % 8 == 0 && a.ccol % 8 == 0 && a.ldo % 8 == 0 && (((uintptr_t)a.proj | (uintptr_t)a.out | (uintptr_t)a.hist) & 15) == 0) {
        const unsigned gy = (unsigned)((a.C / 8 + 255) / 256);
#define NVR_CG(TAPS_)                                                                                                                                \
        do {                                                                                                                                         \
            if (b.T >= 1024) conv_gates8_kernel<TAPS_, 16><<<dim3((unsigned)((b.T + 15) / 16), gy), dim3(256), 0, s>>>(a, b);                         \
            else conv_gates8_kernel<TAPS_, 1><<<dim3((unsigned)b.T, gy), dim3(256), 0, s>>>(a, b);                                                   \
        } while (0)
        if (a.taps == 1) NVR_CG(1); else if (a.taps == 2) NVR_CG(2); else if (a.taps == 3) NVR_CG(3); else NVR_CG(4);
#undef NVR_CG
        return launched("conv_gates");
    }
    const dim3 grid((unsigned)b.T, (unsigned)std::min<int64_t>((a.C + 255) / 256, 16));
    if (bf16) conv_gates_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(a, b);
    else conv_gates_kernel<float><<<grid, dim3(256), 0, s>>>(a, b);
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
    if (bf16 && W % 8 == 0 && ldm % 8 == 0 && (((uintptr_t)m | (uintptr_t)out | (uintptr_t)mu | (uintptr_t)hist) & 15) == 0)
        shift_mixes8_kernel<<<dim3((unsigned)(((int64_t)b.T * (W / 8) + 255) / 256)), dim3(256), 0, s>>>((const bf16_t *)m, ldm, b, (int)W, (int)n, mu, (bf16_t *)out, hist, slots);
    else if (bf16) shift_mixes_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(256), 0, s>>>((const bf16_t *)m, ldm, b, (int)W, (int)n, mu, (bf16_t *)out, hist, slots);
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
