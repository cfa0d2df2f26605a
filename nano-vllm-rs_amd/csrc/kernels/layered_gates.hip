// layered_gates.hip — blocks of pre-norm layers with a layer scale (kernels/layered.h): learned positions, the exponential gates and the read-out of a
// matrix memory (its recurrence is retention's token-gated form, layered.hip), queries / keys / values normed over their projections on their way into the
// pages, an elementwise gated recurrence, the residual joins.  Norms, gates, states and the residual sum are f32 in both operand types.  wave64, gfx950.
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
// sum over the 256 threads of a workgroup; red: 4 floats of LDS; every thread gets the sum
__device__ __forceinline__ float block_sum(float v, float *red) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float log_sigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

int launched(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return nvr::fail(NVR_ERR_HIP, "%s launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

// ------------------------------------------------------------------------------------------------ embedding with learned positions
template <class ET>
__global__ __launch_bounds__(256) void embed_pos_kernel(const ET *__restrict__ E, const ET *__restrict__ P, Batch b, int W, float scale, float *__restrict__ x) {
    const int t = blockIdx.x, sq = b.row_seq[t];
    const int64_t p = b.start[sq] + (t - b.cu[sq]);
    const ET *e = E + b.ids[t] * (int64_t)W;
    float *xr = x + (int64_t)t * W;
    for (int c = threadIdx.x; c < W; c += 256) xr[c] = ld_f(e, c) * scale + (P ? ld_f(P, p * W + c) : 0.f);
}

// ------------------------------------------------------------------------------------------------ exponential gates of a matrix memory
// One workgroup per (sequence, head), 256 rows at a time: every thread computes the two log gates of its row, one thread walks the running maximum through the
// 256 rows (an addition and a maximum per row: the only part that is a recurrence), every thread then takes its row's exponentials.  The arithmetic per row is that
// of a walk row by row, so the result does not depend on where a prompt is cut.
__global__ __launch_bounds__(256) void exp_gates_kernel(const float *__restrict__ pre, int64_t ldp, const float *__restrict__ bi, const float *__restrict__ bfg, float cap, Batch b, int H,
                                                        float *__restrict__ mstate, float *__restrict__ tok_gate, float *__restrict__ floor_out) {
    __shared__ float gis[256], gfs[256], ms[257];
    const int sq = blockIdx.x, h = blockIdx.y;
    const int r0 = b.cu[sq], n = b.cu[sq + 1] - r0;
    float *mst = mstate + (int64_t)b.slot[sq] * H + h;
    if (threadIdx.x == 0) ms[0] = b.start[sq] > 0 ? *mst : 0.f;
    const float vbi = bi[h], vbf = bfg[h], icap = 1.0f / cap;
    for (int i0 = 0; i0 < n; i0 += 256) {
        const int nb = min(256, n - i0), i = threadIdx.x;
        const int64_t t = r0 + i0 + i;
        float gi = 0.f, gf = 0.f;
        if (i < nb) {
            gi = cap * tanhf((pre[t * ldp + h] + vbi) * icap);
            gf = log_sigmoid_f(cap * tanhf((pre[t * ldp + H + h] + vbf) * icap));
            gis[i] = gi; gfs[i] = gf;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            float m = ms[0];
            for (int k = 0; k < nb; ++k) { m = fmaxf(gfs[k] + m, gis[k]); ms[k + 1] = m; }
        }
        __syncthreads();
        if (i < nb) {
            const float mp = ms[i], mn = ms[i + 1];
            tok_gate[(t * H + h) * 2] = expf(gf + mp - mn);
            tok_gate[(t * H + h) * 2 + 1] = expf(gi - mn);
            floor_out[t * H + h] = expf(-mn);
        }
        __syncthreads();
        if (threadIdx.x == 0) ms[0] = ms[nb];
    }
    if (threadIdx.x == 0) *mst = ms[0];       // (thread 0 wrote it last)
}

// one wave per (row, head); heads of up to 256 values are read once and kept in registers
template <class OT>
__global__ __launch_bounds__(256) void memory_readout_kernel(const float *__restrict__ o, const float *__restrict__ floor_in, const OT *__restrict__ gate, int64_t ldg, int64_t gcol, int H,
                                                             int Dv, float eps, const float *__restrict__ w, OT *__restrict__ out, int64_t ldo) {
    const int64_t t = blockIdx.x;
    const int h = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (h >= H) return;
    const float *r = o + (t * H + h) * (int64_t)(Dv + 1);
    float ss = 0.f;
    if (Dv <= 256) {
        float v[4], gt[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {                   // (every load of the wave goes out before the first is used)
            const int c = lane + 64 * k;
            v[k] = c < Dv ? r[c] : 0.f;
            gt[k] = c < Dv ? ld_f(gate, t * ldg + gcol + (int64_t)h * Dv + c) : 0.f;
        }
        const float inv_den = 1.0f / (fmaxf(fabsf(r[Dv]), floor_in[t * H + h]) + 1e-6f);
#pragma unroll
        for (int k = 0; k < 4; ++k) { v[k] *= inv_den; ss += v[k] * v[k]; }
        const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)Dv + eps);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int c = lane + 64 * k;
            const int64_t col = (int64_t)h * Dv + c;
            if (c < Dv) st_f(out, t * ldo + col, v[k] * inv * w[col] * sigmoid_f(gt[k]));
        }
        return;
    }
    const float inv_den = 1.0f / (fmaxf(fabsf(r[Dv]), floor_in[t * H + h]) + 1e-6f);
    for (int c = lane; c < Dv; c += 64) { const float v = r[c] * inv_den; ss += v * v; }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)Dv + eps);
    for (int c = lane; c < Dv; c += 64) {
        const int64_t col = (int64_t)h * Dv + c;
        st_f(out, t * ldo + col, r[c] * inv_den * inv * w[col] * sigmoid_f(ld_f(gate, t * ldg + gcol + col)));
    }
}

// ------------------------------------------------------------------------------------------------ normed queries, keys and values
template <class CT>
__global__ __launch_bounds__(256) void qkv_norm_store_kernel(QkvNormArgs a, Batch b) {
    __shared__ float red[4];
    const int t = blockIdx.x, sq = b.row_seq[t];
    const int p = b.start[sq] + (t - b.cu[sq]);
    const int blk = b.block_tables[(int64_t)sq * b.max_blocks + p / b.block_size], jj = p % b.block_size;
    const int64_t row = (int64_t)blk * b.block_size + jj;
    CT *pr = (CT *)a.proj + (int64_t)t * a.ld;
    const int qn = a.H * a.D, kn = a.G * a.D;
    if (a.wq) {
        float ss = 0.f;
        for (int c = threadIdx.x; c < qn; c += 256) { const float v = ld_f(pr, a.qcol + c); ss += v * v; }
        float f = 1.0f / sqrtf(block_sum(ss, red) / (float)qn + a.eps);
        if (a.temp_every > 0) f *= 1.0f + a.temp_coef * logf((float)((p + 1) / a.temp_every) + 1.0f);
        for (int c = threadIdx.x; c < qn; c += 256) st_f(pr, a.qcol + c, ld_f(pr, a.qcol + c) * f * a.wq[c]);
    }
    CT *kd = (CT *)a.kc + row * kn;
    if (a.wk) {
        float ss = 0.f;
        for (int c = threadIdx.x; c < kn; c += 256) { const float v = ld_f(pr, a.kcol + c); ss += v * v; }
        const float f = 1.0f / sqrtf(block_sum(ss, red) / (float)kn + a.eps);
        for (int c = threadIdx.x; c < kn; c += 256) st_f(kd, c, ld_f(pr, a.kcol + c) * f * a.wk[c]);
    } else
        for (int c = threadIdx.x; c < kn; c += 256) kd[c] = pr[a.kcol + c];
    // values: a wave per key/value head
    const int lane = threadIdx.x & 63, Dv = a.Dv;
    CT *vc = (CT *)a.vc;
    const int64_t grp = ((int64_t)blk * (b.block_size >> 3) + (jj >> 3)) * a.G * Dv;      // grouped pages: [block][block_size / 8][G][Dv][8 keys]
    for (int g = threadIdx.x >> 6; g < a.G; g += 4) {
        float f = 1.f;
        if (a.v_unit) {
            float ss = 0.f;
            for (int c = lane; c < Dv; c += 64) { const float v = ld_f(pr, a.vcol + g * Dv + c); ss += v * v; }
            f = 1.0f / sqrtf(wave_sum(ss) / (float)Dv + a.eps);
        }
        for (int c = lane; c < Dv; c += 64) {
            const float v = ld_f(pr, a.vcol + g * Dv + c) * f;
            if (a.v_grouped) st_f(vc, (grp + g * Dv + c) * 8 + (jj & 7), v);
            else st_f(vc, (row * a.G + g) * Dv + c, v);
        }
    }
}

// The same for 16-bit rows whose parts all start and end at multiples of 8 numbers: 16-byte loads and stores, the two sums of squares in one reduction.
__global__ __launch_bounds__(256) void qkv_norm_store8_kernel(QkvNormArgs a, Batch b) {
    __shared__ float red[8];
    const int t = blockIdx.x, sq = b.row_seq[t];
    const int p = b.start[sq] + (t - b.cu[sq]);
    const int blk = b.block_tables[(int64_t)sq * b.max_blocks + p / b.block_size], jj = p % b.block_size;
    const int64_t row = (int64_t)blk * b.block_size + jj;
    bf16_t *pr = (bf16_t *)a.proj + (int64_t)t * a.ld;
    const int qn = a.H * a.D, kn = a.G * a.D, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float sq2 = 0.f, sk2 = 0.f;
    for (int c = threadIdx.x * 8; c < qn; c += 2048) {
        const uint4 v = *reinterpret_cast<const uint4 *>(pr + a.qcol + c); const bf16_t *e = reinterpret_cast<const bf16_t *>(&v);
#pragma unroll
        for (int k = 0; k < 8; ++k) { const float f = ld_f(e, k); sq2 += f * f; }
    }
    for (int c = threadIdx.x * 8; c < kn; c += 2048) {
        const uint4 v = *reinterpret_cast<const uint4 *>(pr + a.kcol + c); const bf16_t *e = reinterpret_cast<const bf16_t *>(&v);
#pragma unroll
        for (int k = 0; k < 8; ++k) { const float f = ld_f(e, k); sk2 += f * f; }
    }
    sq2 = wave_sum(sq2); sk2 = wave_sum(sk2);
    if (lane == 0) { red[wave] = sq2; red[4 + wave] = sk2; }
    __syncthreads();
    float fq = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)qn + a.eps);
    const float fk = 1.0f / sqrtf(((red[4] + red[5]) + (red[6] + red[7])) / (float)kn + a.eps);
    if (a.temp_every > 0) fq *= 1.0f + a.temp_coef * logf((float)((p + 1) / a.temp_every) + 1.0f);
    for (int c = threadIdx.x * 8; c < qn; c += 2048) {
        uint4 v = *reinterpret_cast<const uint4 *>(pr + a.qcol + c); bf16_t *e = reinterpret_cast<bf16_t *>(&v);
        const float4 w0 = *reinterpret_cast<const float4 *>(a.wq + c), w1 = *reinterpret_cast<const float4 *>(a.wq + c + 4);
        const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
        for (int k = 0; k < 8; ++k) st_f(e, k, ld_f(e, k) * fq * w[k]);
        *reinterpret_cast<uint4 *>(pr + a.qcol + c) = v;
    }
    bf16_t *kd = (bf16_t *)a.kc + row * kn;
    for (int c = threadIdx.x * 8; c < kn; c += 2048) {
        uint4 v = *reinterpret_cast<const uint4 *>(pr + a.kcol + c); bf16_t *e = reinterpret_cast<bf16_t *>(&v);
        const float4 w0 = *reinterpret_cast<const float4 *>(a.wk + c), w1 = *reinterpret_cast<const float4 *>(a.wk + c + 4);
        const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
        for (int k = 0; k < 8; ++k) st_f(e, k, ld_f(e, k) * fk * w[k]);
        *reinterpret_cast<uint4 *>(kd + c) = v;
    }
    // values: 16 lanes of 8 numbers per key/value head and pass (heads of up to 128 numbers in one pass), four heads per wave at a time
    const int Dv = a.Dv, sub = lane >> 4, l16 = lane & 15;
    bf16_t *vc = (bf16_t *)a.vc;
    const int64_t grp = ((int64_t)blk * (b.block_size >> 3) + (jj >> 3)) * a.G * Dv;
    for (int g = wave * 4 + sub; g < (a.G + 15) / 16 * 16; g += 16) {           // (every lane of a wave takes part in the shuffles)
        const bool on = g < a.G;
        float ss = 0.f;
        if (on)
            for (int c = l16 * 8; c < Dv; c += 128) {
                const uint4 v = *reinterpret_cast<const uint4 *>(pr + a.vcol + g * Dv + c); const bf16_t *e = reinterpret_cast<const bf16_t *>(&v);
#pragma unroll
                for (int k = 0; k < 8; ++k) { const float f = ld_f(e, k); ss += f * f; }
            }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
        const float f = a.v_unit ? 1.0f / sqrtf(ss / (float)Dv + a.eps) : 1.f;
        if (on)
            for (int c = l16 * 8; c < Dv; c += 128) {
                uint4 v = *reinterpret_cast<const uint4 *>(pr + a.vcol + g * Dv + c); bf16_t *e = reinterpret_cast<bf16_t *>(&v);
#pragma unroll
                for (int k = 0; k < 8; ++k) st_f(e, k, ld_f(e, k) * f);
                if (a.v_grouped) {
#pragma unroll
                    for (int k = 0; k < 8; ++k) vc[(grp + g * Dv + c + k) * 8 + (jj & 7)] = e[k];
                } else *reinterpret_cast<uint4 *>(vc + (row * a.G + g) * Dv + c) = v;
            }
    }
}

// ------------------------------------------------------------------------------------------------ elementwise gated recurrence
// A workgroup owns 32 channels of one sequence and walks its rows in tiles of 128.  Per tile: all 256 threads turn the projections of the tile's rows into the
// recurrence's coefficients a = 1 - z, b = z cand and the output gate silu(g) (the exponentials do not depend on the state) and leave them in LDS; one
// thread per channel then walks the 128 rows, S <- a S + b, one fused multiply-add per row, leaving S in a's place; all threads write S silu(g).  The walk
// is row by row whatever the portion, so the result does not depend on where a prompt is cut.  FAST (16-bit operands): exponentials and reciprocals on the
// hardware's base-2 units, f32 throughout.
template <bool FAST> __device__ __forceinline__ float sigm(float z) {
    return FAST ? __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * z)) : 1.0f / (1.0f + expf(-z));       // (2^+inf = inf, 1 / inf = 0: no overflow on the way)
}

template <class CT>
__global__ __launch_bounds__(256) void gated_unit_kernel(const CT *__restrict__ proj, int64_t ld, int64_t zcol, int64_t ucol, int64_t gcol, const float *__restrict__ bz,
                                                         const float *__restrict__ bu, Batch b, int N, float *__restrict__ state, CT *__restrict__ out, int64_t ldo) {
    constexpr int CH = 32, R = 128, RG = 256 / CH;
    constexpr bool FAST = sizeof(CT) == 2;
    __shared__ float A[R * CH], Bc[R * CH], Gs[R * CH];
    // consecutive workgroups go to the 8 XCDs in turn: with a grid of a multiple of 8 channel groups, XCD x takes the groups x * (groups / 8) ..., so that the
    // 64-byte pieces of one 128-byte line of a row meet in one L2
    const int ngrp = gridDim.x, bx = (ngrp & 7) == 0 ? (int)(blockIdx.x & 7) * (ngrp >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    const int sq = blockIdx.y, l = threadIdx.x & (CH - 1), rg = threadIdx.x / CH, c = bx * CH + l;
    const bool live = c < N;
    const int r0 = b.cu[sq], n = b.cu[sq + 1] - r0;
    float *sp = state + (int64_t)b.slot[sq] * N + c;
    float S = (live && rg == 0 && b.start[sq] > 0) ? *sp : 0.f;
    const float vbz = live ? bz[c] : 0.f, vbu = live ? bu[c] : 0.f;
    // the projections of a tile's rows are requested one tile ahead, into registers: they arrive while the tile before is walked and written
    CT zr[R / RG], ur[R / RG], gr[R / RG];
    auto request = [&](int i0) {
        const int nb = min(R, n - i0);
#pragma unroll
        for (int k = 0; k < R / RG; ++k) {
            const int r = min(rg + k * RG, nb - 1);
            const CT *pr = proj + (int64_t)(r0 + i0 + r) * ld + c;
            zr[k] = pr[zcol]; ur[k] = pr[ucol]; gr[k] = pr[gcol];
        }
    };
    if (live && n > 0) request(0);
    for (int i0 = 0; i0 < n; i0 += R) {
        const int nb = min(R, n - i0);
        if (live) {
#pragma unroll
            for (int k = 0; k < R / RG; ++k) {
                const int r = rg + k * RG;
                if (r < nb) {
                    const float gg = ld_f(&gr[k], 0), zz = sigm<FAST>(ld_f(&zr[k], 0) + vbz), uu = ld_f(&ur[k], 0) + vbu;
                    const float cand = uu >= 0.f ? uu + 0.5f : sigm<FAST>(uu);
                    A[r * CH + l] = 1.0f - zz; Bc[r * CH + l] = zz * cand; Gs[r * CH + l] = gg * sigm<FAST>(gg);
                }
            }
            if (i0 + R < n) request(i0 + R);
        }
        __syncthreads();
        if (rg == 0 && live) {
            for (int r = 0; r < nb; r += 8) {                // eight rows' coefficients into registers, eight steps, eight stores (rows past nb are read, never used)
                float ca[8], cb[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) { ca[k] = A[(r + k) * CH + l]; cb[k] = Bc[(r + k) * CH + l]; }
#pragma unroll
                for (int k = 0; k < 8; ++k) if (r + k < nb) { S = ca[k] * S + cb[k]; ca[k] = S; }
#pragma unroll
                for (int k = 0; k < 8; ++k) if (r + k < nb) A[(r + k) * CH + l] = ca[k];
            }
        }
        __syncthreads();
        if (live) {
#pragma unroll 4
            for (int r = rg; r < nb; r += RG) st_f(out, (int64_t)(r0 + i0 + r) * ldo + c, A[r * CH + l] * Gs[r * CH + l]);
        }
        __syncthreads();
    }
    if (rg == 0 && live) *sp = S;
}

// ------------------------------------------------------------------------------------------------ residual joins
// One workgroup per row.
template <class YT, bool TWO>
__global__ __launch_bounds__(256) void residual_join_kernel(JoinArgs a) {
    __shared__ float red[4];
    const int64_t t = blockIdx.x;
    const int W = (int)a.W;
    float *xr = a.x + t * W;
    const YT *y1 = (const YT *)a.y1 + t * a.ld1, *y2 = TWO ? (const YT *)a.y2 + t * a.ld2 : nullptr, *ad = a.add ? (const YT *)a.add + t * a.lda : nullptr;
    float f1 = 1.f, f2 = 1.f;
    if (TWO) {
        float s1 = 0.f, s2 = 0.f;
        for (int c = threadIdx.x; c < W; c += 256) { const float u = ld_f(y1, c), v = ld_f(y2, c); s1 += u * u; s2 += v * v; }
        f1 = 1.0f / sqrtf(block_sum(s1, red) / (float)W + a.eps);
        f2 = 1.0f / sqrtf(block_sum(s2, red) / (float)W + a.eps);
    }
    float sn = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) {
        float r = ld_f(y1, c);
        if (TWO) r = 0.5f * (r * f1 * a.w1[c] + ld_f(y2, c) * f2 * a.w2[c]);
        float v = xr[c] + (a.ls ? a.ls[c] * r : r);
        if (ad) v += ld_f(ad, c);
        xr[c] = v; sn += v * v;
    }
    if (a.wn) {
        const float fn = 1.0f / sqrtf(block_sum(sn, red) / (float)W + a.eps);
        YT *o = (YT *)a.out + t * a.ldo;
        for (int c = threadIdx.x; c < W; c += 256) st_f(o, c, xr[c] * fn * a.wn[c]);      // (a thread re-reads what it wrote)
    }
}

template <class CT>
__global__ __launch_bounds__(256) void relu_squared_kernel(const CT *__restrict__ z, int64_t ldz, int64_t T, int64_t F, CT *__restrict__ out, int64_t ldo) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= T * F) return;
    const int64_t t = i / F, c = i - t * F;
    const float v = fmaxf(ld_f(z, t * ldz + c), 0.f);
    st_f(out, t * ldo + c, v * v);
}

// 16-bit rows, 8 numbers per thread (F and both strides multiples of 8, 16-byte aligned rows)
__global__ __launch_bounds__(256) void relu_squared8_kernel(const bf16_t *__restrict__ z, int64_t ldz, int64_t T, int64_t F8, bf16_t *__restrict__ out, int64_t ldo) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= T * F8) return;
    const int64_t t = i / F8, c = (i - t * F8) * 8;
    uint4 v = *reinterpret_cast<const uint4 *>(z + t * ldz + c);
    bf16_t *e = reinterpret_cast<bf16_t *>(&v);
#pragma unroll
    for (int k = 0; k < 8; ++k) { const float r = fmaxf(ld_f(e, k), 0.f); st_f(e, k, r * r); }
    *reinterpret_cast<uint4 *>(out + t * ldo + c) = v;
}

__global__ __launch_bounds__(256) void scale_f32_kernel(float *__restrict__ y, int64_t n, float c) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] *= c;
}

}  // namespace

int embed_pos(const void *E, const void *P, bool bf16, const Batch &b, int64_t W, float scale, float *x, hipStream_t s) {
    if (b.T == 0) return 0;
    if (bf16) embed_pos_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(256), 0, s>>>((const bf16_t *)E, (const bf16_t *)P, b, (int)W, scale, x);
    else embed_pos_kernel<float><<<dim3((unsigned)b.T), dim3(256), 0, s>>>((const float *)E, (const float *)P, b, (int)W, scale, x);
    return launched("embed_pos");
}

int exp_gates(const float *pre, int64_t ldp, const float *bi, const float *bf, float cap, const Batch &b, int64_t H, float *mstate, float *tok_gate, float *floor_out,
              hipStream_t s) {
    if (b.T == 0) return 0;
    if (!(cap > 0.f)) return nvr::fail(NVR_ERR_INVALID_ARG, "exp_gates: the gates' cap must be positive");
    exp_gates_kernel<<<dim3((unsigned)b.B, (unsigned)H), dim3(256), 0, s>>>(pre, ldp, bi, bf, cap, b, (int)H, mstate, tok_gate, floor_out);
    return launched("exp_gates");
}

int memory_readout(const float *o, const float *floor_in, const void *gate, int64_t ldg, int64_t gcol, int64_t T, int64_t H, int64_t Dv, float eps, const float *w, void *out,
                   int64_t ldo, bool bf16, hipStream_t s) {
    if (T == 0) return 0;
    const dim3 grid((unsigned)T, (unsigned)((H + 3) / 4));
    if (bf16) memory_readout_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(o, floor_in, (const bf16_t *)gate, ldg, gcol, (int)H, (int)Dv, eps, w, (bf16_t *)out, ldo);
    else memory_readout_kernel<float><<<grid, dim3(256), 0, s>>>(o, floor_in, (const float *)gate, ldg, gcol, (int)H, (int)Dv, eps, w, (float *)out, ldo);
    return launched("memory_readout");
}

int qkv_norm_store(const QkvNormArgs &a, const Batch &b, bool bf16, hipStream_t s) {
    if (b.T == 0) return 0;
    if (a.v_grouped && b.block_size % 8) return nvr::fail(NVR_ERR_INVALID_ARG, "qkv_norm_store: grouped value pages need pages of a multiple of 8 tokens");
    const bool vec = bf16 && a.wq && a.wk && a.D % 8 == 0 && a.Dv % 8 == 0 && a.ld % 8 == 0 && ((a.qcol | a.kcol | a.vcol) & 7) == 0 &&
                     (((uintptr_t)a.proj | (uintptr_t)a.kc | (uintptr_t)a.vc | (uintptr_t)a.wq | (uintptr_t)a.wk) & 15) == 0;
    if (vec) qkv_norm_store8_kernel<<<dim3((unsigned)b.T), dim3(256), 0, s>>>(a, b);
    else if (bf16) qkv_norm_store_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(256), 0, s>>>(a, b);
    else qkv_norm_store_kernel<float><<<dim3((unsigned)b.T), dim3(256), 0, s>>>(a, b);
    return launched("qkv_norm_store");
}

int gated_unit(const void *proj, int64_t ld, int64_t zcol, int64_t ucol, int64_t gcol, const float *bz, const float *bu, const Batch &b, int64_t N, float *state, void *out, int64_t ldo,
               bool bf16, hipStream_t s) {
    if (b.T == 0 || N == 0) return 0;
    const dim3 grid((unsigned)((N + 31) / 32), (unsigned)b.B);
    if (bf16) gated_unit_kernel<bf16_t><<<grid, dim3(256), 0, s>>>((const bf16_t *)proj, ld, zcol, ucol, gcol, bz, bu, b, (int)N, state, (bf16_t *)out, ldo);
    else gated_unit_kernel<float><<<grid, dim3(256), 0, s>>>((const float *)proj, ld, zcol, ucol, gcol, bz, bu, b, (int)N, state, (float *)out, ldo);
    return launched("gated_unit");
}

int residual_join(const JoinArgs &a, bool bf16, hipStream_t s) {
    if (a.T == 0) return 0;
    if (a.y2 && (!a.w1 || !a.w2)) return nvr::fail(NVR_ERR_INVALID_ARG, "residual_join: two branches need their norms' weights");
    const dim3 grid((unsigned)a.T);
    if (a.y2) { if (bf16) residual_join_kernel<bf16_t, true><<<grid, dim3(256), 0, s>>>(a); else residual_join_kernel<float, true><<<grid, dim3(256), 0, s>>>(a); }
    else { if (bf16) residual_join_kernel<bf16_t, false><<<grid, dim3(256), 0, s>>>(a); else residual_join_kernel<float, false><<<grid, dim3(256), 0, s>>>(a); }
    return launched("residual_join");
}

int relu_squared(const void *z, int64_t ldz, int64_t T, int64_t F, void *out, int64_t ldo, bool bf16, hipStream_t s) {
    if (T * F == 0) return 0;
    if (bf16 && F % 8 == 0 && ldz % 8 == 0 && ldo % 8 == 0 && (((uintptr_t)z | (uintptr_t)out) & 15) == 0) {
        relu_squared8_kernel<<<dim3((unsigned)((T * (F / 8) + 255) / 256)), dim3(256), 0, s>>>((const bf16_t *)z, ldz, T, F / 8, (bf16_t *)out, ldo);
        return launched("relu_squared");
    }
    const dim3 grid((unsigned)((T * F + 255) / 256));
    if (bf16) relu_squared_kernel<bf16_t><<<grid, dim3(256), 0, s>>>((const bf16_t *)z, ldz, T, F, (bf16_t *)out, ldo);
    else relu_squared_kernel<float><<<grid, dim3(256), 0, s>>>((const float *)z, ldz, T, F, (float *)out, ldo);
    return launched("relu_squared");
}

int scale_f32(float *y, int64_t n, float c, hipStream_t s) {
    if (n == 0) return 0;
    scale_f32_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s>>>(y, n, c);
    return launched("scale_f32");
}

}}  // namespace nvr::kl
