// layered_blocks.hip — further building blocks of layer-list models (kernels/layered.h): RMS norm in groups with a weight (alone, added to the
// residual stream, and followed by the next sublayer's norm), the cached row of latent attention (normed latent + rotated shared key part), products
// with one small matrix per head (absorbing the key expansion into the query, expanding values), the polynomial-norm activation, a mixture of
// experts (sigmoid router, top-k, rows grouped by expert, one grouped product per projection), the per-layer token input and the weighted
// average over the depth of the stack.  wave64, gfx950.  Norms, routers, angles and the residual sum are f32 in both operand types.
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
__device__ __forceinline__ float block_sum256(float v, float *red) {       // red: 4 floats of LDS
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float gelu_tanh_f(float z) { return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }

int launched(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return nvr::fail(NVR_ERR_HIP, "%s launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

// ------------------------------------------------------------------------------------------------ RMS norm in groups
// One workgroup per row, a wave per group (groups beyond four in turns).  IT: type of the input rows.  ADD: the normed row is added to the f32 row xres (the
// sublayer's output joining the residual stream) instead of being stored; with w2 the new residual row is normed once more into out (the next sublayer's input).
template <class IT, class OT, bool ADD>
__global__ __launch_bounds__(256) void group_norm_kernel(const IT *__restrict__ in, int64_t ldi, const int32_t *__restrict__ rows, int W, int groups, float eps,
                                                         const float *__restrict__ w, float *__restrict__ xres, const float *__restrict__ w2, int plain,
                                                         OT *__restrict__ out, int64_t ldo) {
    const int64_t r = blockIdx.x, src = rows ? rows[r] : r;
    const IT *x = in + src * ldi;
    const int n = W / groups, lane = threadIdx.x & 63;
    for (int g = threadIdx.x >> 6; g < groups; g += 4) {
        const int c0 = g * n;
        float ss = 0.f;
        for (int c = lane; c < n; c += 64) { const float v = ld_f(x, c0 + c); ss += v * v; }
        const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)n + eps);
        if (!ADD) {
            for (int c = lane; c < n; c += 64) st_f(out, r * ldo + c0 + c, ld_f(x, c0 + c) * inv * w[c0 + c]);
        } else {
            float *xr = xres + r * (int64_t)W;
            float s2 = 0.f;
            for (int c = lane; c < n; c += 64) {
                const float v = xr[c0 + c] + ld_f(x, c0 + c) * inv * w[c0 + c];
                xr[c0 + c] = v; s2 += v * v;
                if (plain) st_f(out, r * ldo + c0 + c, v);
            }
            if (w2) {
                const float inv2 = 1.0f / sqrtf(wave_sum(s2) / (float)n + eps);
                for (int c = lane; c < n; c += 64) st_f(out, r * ldo + c0 + c, xr[c0 + c] * inv2 * w2[c0 + c]);   // (a lane re-reads what it wrote)
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------ the cached row of latent attention
// Row t of proj holds, from column col, `rank` latent numbers and `rot` numbers of the shared key part.  The page row of the token's position receives the latent
// divided by its root mean square times w, and the key part with coordinate pairs (2i, 2i+1) turned by position * freq[i].
template <class CT>
__global__ __launch_bounds__(64) void latent_store_kernel(const CT *__restrict__ proj, int64_t ld, int64_t col, Batch b, int rank, int rot, float eps,
                                                          const float *__restrict__ w, const float *__restrict__ freq, CT *__restrict__ pages, CT *__restrict__ rows) {
    const int t = blockIdx.x, sq = b.row_seq[t], lane = threadIdx.x;
    const int p = b.start[sq] + (t - b.cu[sq]);
    const int blk = b.block_tables[(int64_t)sq * b.max_blocks + p / b.block_size];
    CT *dst = pages + ((int64_t)blk * b.block_size + p % b.block_size) * (rank + rot);
    const CT *src = proj + (int64_t)t * ld + col;
    float ss = 0.f;
    for (int c = lane; c < rank; c += 64) { const float v = ld_f(src, c); ss += v * v; }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)rank + eps);
    CT *dst2 = rows ? rows + (int64_t)t * (rank + rot) : nullptr;      // the same row once more, in step order
    for (int c = lane; c < rank; c += 64) { const float v = ld_f(src, c) * inv * w[c]; st_f(dst, c, v); if (dst2) st_f(dst2, c, v); }
    for (int i = lane; i < rot / 2; i += 64) {
        const float ang = (float)p * freq[i], cs = cosf(ang), sn = sinf(ang);
        const float u = ld_f(src, rank + 2 * i), v = ld_f(src, rank + 2 * i + 1);
        st_f(dst, rank + 2 * i, u * cs - v * sn); st_f(dst, rank + 2 * i + 1, v * cs + u * sn);
        if (dst2) { st_f(dst2, rank + 2 * i, u * cs - v * sn); st_f(dst2, rank + 2 * i + 1, v * cs + u * sn); }
    }
}

// q rows [H][D + rot]: the last rot numbers of every head, rotated like the key part, go to out rows [H][ldh] at column ocol
template <class CT>
__global__ __launch_bounds__(256) void rotate_heads_kernel(const CT *__restrict__ q, int64_t ldq, int qstride, int qcol, Batch b, int H, int rot, const float *__restrict__ freq,
                                                           CT *__restrict__ out, int64_t ldo, int ostride, int ocol) {
    const int t = blockIdx.x, sq = b.row_seq[t];
    const int p = b.start[sq] + (t - b.cu[sq]);
    const int half = rot / 2;
    for (int idx = threadIdx.x; idx < H * half; idx += 256) {
        const int h = idx / half, i = idx - h * half;
        const float ang = (float)p * freq[i], cs = cosf(ang), sn = sinf(ang);
        const CT *src = q + (int64_t)t * ldq + (int64_t)h * qstride + qcol;
        const float u = ld_f(src, 2 * i), v = ld_f(src, 2 * i + 1);
        CT *dst = out + (int64_t)t * ldo + (int64_t)h * ostride + ocol;
        st_f(dst, 2 * i, u * cs - v * sn); st_f(dst, 2 * i + 1, v * cs + u * sn);
    }
}

// ------------------------------------------------------------------------------------------------ one small matrix per head / per group of rows
// A 64 x 64 tile of y = a . w^T per workgroup, K in steps of 16 through LDS, 4 x 4 outputs per thread, f32 accumulation.
struct TileJob {
    const void *a; int64_t lda; const void *w; int64_t ldw; void *y; int64_t ldy;
    int rows, K, N;                               // this job's extent
    const void *gate; int64_t ldg;                // y *= sigmoid(gate) (same row / column as y) when not null
    const int32_t *src; const float *rscale; int src_div;   // row r of a is row src[r] / src_div of the array, times rscale[src[r]], when src is not null
};
template <class ET>
__device__ __forceinline__ void tile_product(const TileJob &j, int row0, int col0, float (*As)[68], float (*Ws)[68]) {
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const ET *a = (const ET *)j.a; const ET *w = (const ET *)j.w;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < j.K; k0 += 16) {
        for (int idx = threadIdx.x; idx < 64 * 16; idx += 256) {
            const int r = idx >> 4, k = idx & 15;
            float av = 0.f, wv = 0.f;
            if (row0 + r < j.rows && k0 + k < j.K) {
                if (j.src) { const int sidx = j.src[row0 + r]; av = ld_f(a, (int64_t)(sidx / j.src_div) * j.lda + k0 + k) * j.rscale[sidx]; }
                else av = ld_f(a, (int64_t)(row0 + r) * j.lda + k0 + k);
            }
            if (col0 + r < j.N && k0 + k < j.K) wv = ld_f(w, (int64_t)(col0 + r) * j.ldw + k0 + k);
            if (sizeof(ET) == 2 && j.src) { bf16_t h; st_f(&h, 0, av); av = ld_f(&h, 0); }     // (the scaled row is an operand: one rounding, as a stored copy would have)
            As[k][r] = av; Ws[k][r] = wv;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { av[i] = As[k][ty * 4 + i]; wv[i] = Ws[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[i][c] = fmaf(av[i], wv[c], acc[i][c]);
        }
        __syncthreads();
    }
    ET *y = (ET *)j.y;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int r = row0 + ty * 4 + i, n = col0 + tx * 4 + c;
            if (r < j.rows && n < j.N) {
                float v = acc[i][c];
                if (j.gate) v *= sigmoid_f(ld_f((const ET *)j.gate, (int64_t)r * j.ldg + n));
                st_f(y, (int64_t)r * j.ldy + n, v);
            }
        }
}

// The same on the matrix cores for bfloat16 operands (K a multiple of 8, rows 16-byte aligned): v_mfma_f32_16x16x32_bf16, fragments straight from global
// memory (a lane's 8 consecutive k of its row / column are one 16-byte load; nothing staged in LDS, no barrier).  WR = 4: the four waves take 16 rows each of
// a 64 x 64 tile; WR = 1: they take 64 columns each of a 16 x 256 tile (few rows: decode-sized steps, experts with few tokens).
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int WR>
__device__ __forceinline__ void tile_product_mfma(const TileJob &j, int row0, int col0) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lm = lane & 15, lq = lane >> 4;
    const int rbase = row0 + (WR == 4 ? wave * 16 : 0), cbase = col0 + (WR == 4 ? 0 : wave * 64);
    if (rbase >= j.rows || cbase >= j.N) return;
    const bf16_t *w = (const bf16_t *)j.w;
    const int r = rbase + lm;
    const bool rok = r < j.rows;
    const bf16_t *ap = (const bf16_t *)j.a; float rs = 1.f;
    if (rok) {
        if (j.src) { const int sidx = j.src[r]; ap += (int64_t)(sidx / j.src_div) * j.lda; rs = j.rscale[sidx]; }
        else ap += (int64_t)r * j.lda;
    }
    const bf16_t *wp[4]; bool cok[4];
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) { const int n = cbase + cb * 16 + lm; cok[cb] = n < j.N; wp[cb] = w + (int64_t)(cok[cb] ? n : 0) * j.ldw; }
    f32x4 acc[4];
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) acc[cb] = f32x4{0.f, 0.f, 0.f, 0.f};
    const uint4 zero{0, 0, 0, 0};
#pragma unroll 2
    for (int k0 = 0; k0 < j.K; k0 += 32) {
        const int k = k0 + lq * 8;
        const bool kok = k < j.K;
        uint4 av = (rok && kok) ? *reinterpret_cast<const uint4 *>(ap + k) : zero;
        uint4 wv[4];
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) wv[cb] = (cok[cb] && kok) ? *reinterpret_cast<const uint4 *>(wp[cb] + k) : zero;
        if (j.src) {                                        // the scaled row is an operand: one rounding, as a stored copy would have
            bf16_t *e = reinterpret_cast<bf16_t *>(&av);
#pragma unroll
            for (int y = 0; y < 8; ++y) st_f(e, y, ld_f(e, y) * rs);
        }
        const bf16x8 af = __builtin_bit_cast(bf16x8, av);
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, __builtin_bit_cast(bf16x8, wv[cb]), acc[cb], 0, 0, 0);
    }
    bf16_t *y = (bf16_t *)j.y;
#pragma unroll
    for (int cb = 0; cb < 4; ++cb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int rr = rbase + lq * 4 + i, n = cbase + cb * 16 + lm;
            if (rr < j.rows && n < j.N) {
                float v = acc[cb][i];
                if (j.gate) v *= sigmoid_f(ld_f((const bf16_t *)j.gate, (int64_t)rr * j.ldg + n));
                st_f(y, (int64_t)rr * j.ldy + n, v);
            }
        }
}

// Many rows: a 128 x 128 tile per workgroup, K in steps of 64 through LDS (the next step's 16-byte pieces are requested before the current step's
// arithmetic); the four waves own 64 x 64 quarters, 32 MFMAs per step.
__device__ __forceinline__ void tile_product_mfma128(const TileJob &j, int row0, int col0, bf16_t *As, bf16_t *Ws) {
    constexpr int KS = 64, LD = KS + 8;                     // rows stay 16-byte aligned and spread over the banks
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lm = lane & 15, lq = lane >> 4, wr = wave >> 1, wc = wave & 1;
    const int lrow = threadIdx.x >> 3, lch = threadIdx.x & 7;
    const bf16_t *ap[4], *wp[4]; bool aok[4], wok[4]; float rs[4] = {1.f, 1.f, 1.f, 1.f};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int r = row0 + lrow + 32 * q, n = col0 + lrow + 32 * q;
        aok[q] = r < j.rows; wok[q] = n < j.N;
        ap[q] = (const bf16_t *)j.a; wp[q] = (const bf16_t *)j.w + (int64_t)(wok[q] ? n : 0) * j.ldw;
        if (aok[q]) {
            if (j.src) { const int sidx = j.src[r]; ap[q] += (int64_t)(sidx / j.src_div) * j.lda; rs[q] = j.rscale[sidx]; }
            else ap[q] += (int64_t)r * j.lda;
        }
    }
    f32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[i][c] = f32x4{0.f, 0.f, 0.f, 0.f};
    const uint4 zero{0, 0, 0, 0};
    uint4 ra[4], rw[4];
    auto fetch = [&](int k0) {
        const int k = k0 + lch * 8;
        const bool kok = k < j.K;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            ra[q] = (aok[q] && kok) ? *reinterpret_cast<const uint4 *>(ap[q] + k) : zero;
            rw[q] = (wok[q] && kok) ? *reinterpret_cast<const uint4 *>(wp[q] + k) : zero;
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < j.K; k0 += KS) {
        if (j.src) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                bf16_t *e = reinterpret_cast<bf16_t *>(&ra[q]);
#pragma unroll
                for (int y = 0; y < 8; ++y) st_f(e, y, ld_f(e, y) * rs[q]);
            }
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            *reinterpret_cast<uint4 *>(As + (lrow + 32 * q) * LD + lch * 8) = ra[q];
            *reinterpret_cast<uint4 *>(Ws + (lrow + 32 * q) * LD + lch * 8) = rw[q];
        }
        __syncthreads();
        if (k0 + KS < j.K) fetch(k0 + KS);
#pragma unroll
        for (int kk = 0; kk < KS; kk += 32) {
            bf16x8 af[4], wf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                af[i] = *reinterpret_cast<const bf16x8 *>(As + (wr * 64 + i * 16 + lm) * LD + kk + lq * 8);
                wf[i] = *reinterpret_cast<const bf16x8 *>(Ws + (wc * 64 + i * 16 + lm) * LD + kk + lq * 8);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[i][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], wf[c], acc[i][c], 0, 0, 0);
        }
    }
    bf16_t *y = (bf16_t *)j.y;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int rr = row0 + wr * 64 + i * 16 + lq * 4 + e, n = col0 + wc * 64 + c * 16 + lm;
                if (rr < j.rows && n < j.N) {
                    float v = acc[i][c][e];
                    if (j.gate) v *= sigmoid_f(ld_f((const bf16_t *)j.gate, (int64_t)rr * j.ldg + n));
                    st_f(y, (int64_t)rr * j.ldy + n, v);
                }
            }
}

__global__ __launch_bounds__(256) void head_linear_mfma128_kernel(HeadLinearArgs p) {
    __shared__ __attribute__((aligned(16))) bf16_t As[128 * 72], Ws[128 * 72];
    const int h = blockIdx.z;
    TileJob j{};
    j.a = (const bf16_t *)p.a + (int64_t)h * p.ha; j.lda = p.lda; j.w = (const bf16_t *)p.w + (int64_t)h * p.N * p.K; j.ldw = p.K;
    j.y = (bf16_t *)p.y + (int64_t)h * p.hy; j.ldy = p.ldy; j.rows = p.T; j.K = p.K; j.N = p.N;
    j.gate = p.gate ? (const void *)((const bf16_t *)p.gate + (int64_t)h * p.hg) : nullptr; j.ldg = p.ldg;
    tile_product_mfma128(j, blockIdx.y * 128, blockIdx.x * 128, As, Ws);
}

__global__ __launch_bounds__(256) void grouped_linear_mfma128_kernel(GroupedLinearArgs p) {
    __shared__ __attribute__((aligned(16))) bf16_t As[128 * 72], Ws[128 * 72];
    int tile = blockIdx.y, e = 0, lo = 0, hi = 0;
    for (; e < p.groups; ++e) {
        lo = p.off[e]; hi = p.off[e + 1];
        const int nt = (hi - lo + 127) >> 7;
        if (tile < nt) break;
        tile -= nt;
    }
    if (e == p.groups) return;                              // (every thread of the workgroup leaves: no barrier is left waiting)
    TileJob j{};
    j.lda = p.lda; j.w = (const bf16_t *)p.w + (int64_t)e * p.N * p.K; j.ldw = p.K; j.y = (bf16_t *)p.y + (int64_t)lo * p.ldy; j.ldy = p.ldy;
    j.rows = hi - lo; j.K = p.K; j.N = p.N;
    if (p.src) { j.a = p.a; j.src = p.src + lo; j.rscale = p.rscale; j.src_div = p.src_div; }
    else j.a = (const bf16_t *)p.a + (int64_t)lo * p.lda;
    tile_product_mfma128(j, tile * 128, blockIdx.x * 128, As, Ws);
}

// Few rows (decode-sized steps, experts with a handful of tokens): a 16 x 64 tile per workgroup and the four waves split K, so that a product whose cost is
// reading the matrix is spread over four times as many workgroups; the partial sums meet in LDS.
__device__ __forceinline__ void tile_product_mfma_ksplit(const TileJob &j, int row0, int col0, float *part) {      // part: [3][16 * 64] floats of LDS
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lm = lane & 15, lq = lane >> 4;
    const bf16_t *w = (const bf16_t *)j.w;
    const int r = row0 + lm;
    const bool rok = r < j.rows;
    const bf16_t *ap = (const bf16_t *)j.a; float rs = 1.f;
    if (rok) {
        if (j.src) { const int sidx = j.src[r]; ap += (int64_t)(sidx / j.src_div) * j.lda; rs = j.rscale[sidx]; }
        else ap += (int64_t)r * j.lda;
    }
    const bf16_t *wp[4]; bool cok[4];
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) { const int n = col0 + cb * 16 + lm; cok[cb] = n < j.N; wp[cb] = w + (int64_t)(cok[cb] ? n : 0) * j.ldw; }
    f32x4 acc[4];
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) acc[cb] = f32x4{0.f, 0.f, 0.f, 0.f};
    const uint4 zero{0, 0, 0, 0};
    const int kq = ((j.K + 3) / 4 + 31) / 32 * 32, kbeg = wave * kq, kend = min(j.K, kbeg + kq);
#pragma unroll 2
    for (int k0 = kbeg; k0 < kend; k0 += 32) {
        const int k = k0 + lq * 8;
        const bool kok = k < kend;
        uint4 av = (rok && kok) ? *reinterpret_cast<const uint4 *>(ap + k) : zero;
        uint4 wv[4];
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) wv[cb] = (cok[cb] && kok) ? *reinterpret_cast<const uint4 *>(wp[cb] + k) : zero;
        if (j.src) {
            bf16_t *e = reinterpret_cast<bf16_t *>(&av);
#pragma unroll
            for (int y = 0; y < 8; ++y) st_f(e, y, ld_f(e, y) * rs);
        }
        const bf16x8 af = __builtin_bit_cast(bf16x8, av);
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, __builtin_bit_cast(bf16x8, wv[cb]), acc[cb], 0, 0, 0);
    }
    if (wave > 0)
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
#pragma unroll
            for (int i = 0; i < 4; ++i) part[(wave - 1) * 1024 + (lq * 4 + i) * 64 + cb * 16 + lm] = acc[cb][i];
    __syncthreads();
    if (wave > 0) return;
    bf16_t *y = (bf16_t *)j.y;
#pragma unroll
    for (int cb = 0; cb < 4; ++cb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int rr = row0 + lq * 4 + i, n = col0 + cb * 16 + lm, at = (lq * 4 + i) * 64 + cb * 16 + lm;
            if (rr < j.rows && n < j.N) {
                float v = (acc[cb][i] + part[at]) + (part[1024 + at] + part[2048 + at]);
                if (j.gate) v *= sigmoid_f(ld_f((const bf16_t *)j.gate, (int64_t)rr * j.ldg + n));
                st_f(y, (int64_t)rr * j.ldy + n, v);
            }
        }
}

__global__ __launch_bounds__(256) void head_linear_ksplit_kernel(HeadLinearArgs p) {
    __shared__ float part[3 * 1024];
    const int h = blockIdx.z;
    TileJob j{};
    j.a = (const bf16_t *)p.a + (int64_t)h * p.ha; j.lda = p.lda; j.w = (const bf16_t *)p.w + (int64_t)h * p.N * p.K; j.ldw = p.K;
    j.y = (bf16_t *)p.y + (int64_t)h * p.hy; j.ldy = p.ldy; j.rows = p.T; j.K = p.K; j.N = p.N;
    j.gate = p.gate ? (const void *)((const bf16_t *)p.gate + (int64_t)h * p.hg) : nullptr; j.ldg = p.ldg;
    tile_product_mfma_ksplit(j, blockIdx.y * 16, blockIdx.x * 64, part);
}

__global__ __launch_bounds__(256) void grouped_linear_ksplit_kernel(GroupedLinearArgs p) {
    __shared__ float part[3 * 1024];
    int tile = blockIdx.y, e = 0, lo = 0, hi = 0;
    for (; e < p.groups; ++e) {
        lo = p.off[e]; hi = p.off[e + 1];
        const int nt = (hi - lo + 15) >> 4;
        if (tile < nt) break;
        tile -= nt;
    }
    if (e == p.groups) return;                              // (the whole workgroup leaves)
    TileJob j{};
    j.lda = p.lda; j.w = (const bf16_t *)p.w + (int64_t)e * p.N * p.K; j.ldw = p.K; j.y = (bf16_t *)p.y + (int64_t)lo * p.ldy; j.ldy = p.ldy;
    j.rows = hi - lo; j.K = p.K; j.N = p.N;
    if (p.src) { j.a = p.a; j.src = p.src + lo; j.rscale = p.rscale; j.src_div = p.src_div; }
    else j.a = (const bf16_t *)p.a + (int64_t)lo * p.lda;
    tile_product_mfma_ksplit(j, tile * 16, blockIdx.x * 64, part);
}

template <int WR>
__global__ __launch_bounds__(256) void head_linear_mfma_kernel(HeadLinearArgs p) {
    const int h = blockIdx.z;
    TileJob j{};
    j.a = (const bf16_t *)p.a + (int64_t)h * p.ha; j.lda = p.lda; j.w = (const bf16_t *)p.w + (int64_t)h * p.N * p.K; j.ldw = p.K;
    j.y = (bf16_t *)p.y + (int64_t)h * p.hy; j.ldy = p.ldy; j.rows = p.T; j.K = p.K; j.N = p.N;
    j.gate = p.gate ? (const void *)((const bf16_t *)p.gate + (int64_t)h * p.hg) : nullptr; j.ldg = p.ldg;
    tile_product_mfma<WR>(j, blockIdx.y * (WR * 16), blockIdx.x * (WR == 4 ? 64 : 256));
}

template <int WR>
__global__ __launch_bounds__(256) void grouped_linear_mfma_kernel(GroupedLinearArgs p) {
    constexpr int TR = WR * 16;
    int tile = blockIdx.y, e = 0, lo = 0, hi = 0;
    for (; e < p.groups; ++e) {
        lo = p.off[e]; hi = p.off[e + 1];
        const int nt = (hi - lo + TR - 1) / TR;
        if (tile < nt) break;
        tile -= nt;
    }
    if (e == p.groups) return;
    TileJob j{};
    j.lda = p.lda; j.w = (const bf16_t *)p.w + (int64_t)e * p.N * p.K; j.ldw = p.K; j.y = (bf16_t *)p.y + (int64_t)lo * p.ldy; j.ldy = p.ldy;
    j.rows = hi - lo; j.K = p.K; j.N = p.N;
    if (p.src) { j.a = p.a; j.src = p.src + lo; j.rscale = p.rscale; j.src_div = p.src_div; }
    else j.a = (const bf16_t *)p.a + (int64_t)lo * p.lda;
    tile_product_mfma<WR>(j, tile * TR, blockIdx.x * (WR == 4 ? 64 : 256));
}

// y[t][h][n] = sum_k a[t][h][k] w[h][n][k]: blockIdx.z is the head
template <class ET>
__global__ __launch_bounds__(256) void head_linear_kernel(HeadLinearArgs p) {
    __shared__ float As[16][68], Ws[16][68];
    const int h = blockIdx.z;
    TileJob j{};
    j.a = (const ET *)p.a + (int64_t)h * p.ha; j.lda = p.lda; j.w = (const ET *)p.w + (int64_t)h * p.N * p.K; j.ldw = p.K;
    j.y = (ET *)p.y + (int64_t)h * p.hy; j.ldy = p.ldy; j.rows = p.T; j.K = p.K; j.N = p.N;
    j.gate = p.gate ? (const void *)((const ET *)p.gate + (int64_t)h * p.hg) : nullptr; j.ldg = p.ldg;
    tile_product<ET>(j, blockIdx.y * 64, blockIdx.x * 64, As, Ws);
}

// Rows grouped by expert: group e owns rows off[e] .. off[e+1]-1 and the matrix w[e] ([N][K]).  blockIdx.y walks the row tiles of all groups (at most
// rows / 64 + groups of them); a workgroup finds its group by walking the offsets, and leaves when it is beyond the last tile.
template <class ET>
__global__ __launch_bounds__(256) void grouped_linear_kernel(GroupedLinearArgs p) {
    __shared__ float As[16][68], Ws[16][68];
    int tile = blockIdx.y, e = 0, lo = 0, hi = 0;
    for (; e < p.groups; ++e) {
        lo = p.off[e]; hi = p.off[e + 1];
        const int nt = (hi - lo + 63) >> 6;
        if (tile < nt) break;
        tile -= nt;
    }
    if (e == p.groups) return;
    TileJob j{};
    j.lda = p.lda; j.w = (const ET *)p.w + (int64_t)e * p.N * p.K; j.ldw = p.K; j.y = (ET *)p.y + (int64_t)lo * p.ldy; j.ldy = p.ldy;
    j.rows = hi - lo; j.K = p.K; j.N = p.N;
    if (p.src) { j.a = p.a; j.src = p.src + lo; j.rscale = p.rscale; j.src_div = p.src_div; }
    else j.a = (const ET *)p.a + (int64_t)lo * p.lda;
    tile_product<ET>(j, tile * 64, blockIdx.x * 64, As, Ws);
}

// ------------------------------------------------------------------------------------------------ activations
// out = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3 with N(v) = v / sqrt(mean(v^2) + eps) over the row
template <class OT>
__global__ __launch_bounds__(256) void poly_norm_kernel(const OT *__restrict__ z, int64_t ldz, int F, float eps, const float *__restrict__ coef, OT *__restrict__ out, int64_t ldo) {
    __shared__ float red[4];
    const int64_t t = blockIdx.x;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int c = threadIdx.x; c < F; c += 256) { const float v = ld_f(z, t * ldz + c), v2 = v * v; s1 += v2; s2 += v2 * v2; s3 += v2 * v2 * v2; }
    s1 = block_sum256(s1, red); s2 = block_sum256(s2, red); s3 = block_sum256(s3, red);
    const float i1 = coef[0] / sqrtf(s1 / (float)F + eps), i2 = coef[1] / sqrtf(s2 / (float)F + eps), i3 = coef[2] / sqrtf(s3 / (float)F + eps), e = coef[3];
    for (int c = threadIdx.x; c < F; c += 256) { const float v = ld_f(z, t * ldz + c); st_f(out, t * ldo + c, v * i1 + v * v * i2 + v * v * v * i3 + e); }
}

// out = silu(gate) * up; gu rows [2 F] (gate columns, then up columns)
template <class OT>
__global__ __launch_bounds__(256) void silu_mul_kernel(const OT *__restrict__ gu, int64_t T, int64_t F, OT *__restrict__ out, int64_t ldo) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= T * F) return;
    const int64_t t = idx / F, c = idx - t * F;
    const float g = ld_f(gu, t * 2 * F + c);
    st_f(out, t * ldo + c, g * sigmoid_f(g) * ld_f(gu, t * 2 * F + F + c));
}

// ------------------------------------------------------------------------------------------------ mixture of experts
// Router: z = Wr h in f32; the `top` largest logits of a token (the lower index wins a tie) go to sel, their sigmoid to score ([T][top]).  The logits and not the
// scores are compared: the order is the same, and saturated scores do not tie.  softmax: the score of a chosen expert is its share e^(z - max) / sum over ALL experts,
// divided by the sum of the chosen shares (+ 1e-20).  Rows E .. E + extra - 1 of wr are further projections of h whose values leave as they are.
template <class OT>
__global__ __launch_bounds__(256) void moe_route_kernel(const OT *__restrict__ h, int64_t ldh, int W, const float *__restrict__ wr, int E, int top,
                                                        int32_t *__restrict__ sel, float *__restrict__ score, int softmax, int extra, float *__restrict__ extra_out,
                                                        const float *__restrict__ logits, int64_t ldl) {
    extern __shared__ float sc[];                       // [E + extra]
    const int64_t t = blockIdx.x; const int lane = threadIdx.x & 63;
    if (logits)                                         // the products were formed by a matrix product before this launch
        for (int e = threadIdx.x; e < E + extra; e += 256) { const float d = logits[t * ldl + e]; sc[e] = d; if (e >= E) extra_out[t * extra + (e - E)] = d; }
    else
    for (int e = threadIdx.x >> 6; e < E + extra; e += 4) {
        float d = 0.f;
        for (int c = lane; c < W; c += 64) d = fmaf(ld_f(h, t * ldh + c), wr[(int64_t)e * W + c], d);
        d = wave_sum(d);
        if (lane == 0) { sc[e] = d; if (e >= E) extra_out[t * extra + (e - E)] = d; }
    }
    __syncthreads();
    float zmax = 0.f, zsum = 1.f;
    if (softmax && threadIdx.x < 64) {                  // (the first wave keeps both for its choices below)
        zmax = -INFINITY;
        for (int e = lane; e < E; e += 64) zmax = fmaxf(zmax, sc[e]);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) zmax = fmaxf(zmax, __shfl_xor(zmax, o, 64));
        zsum = 0.f;
        for (int e = lane; e < E; e += 64) zsum += expf(sc[e] - zmax);
        zsum = wave_sum(zsum);
    }
    float chosen = 0.f;                                 // (lane 0: the sum of the chosen shares)
    for (int k = 0; k < top; ++k) {                     // the first wave: top times the arg-max over the experts' logits
        if (threadIdx.x < 64) {
            float best = -INFINITY; int bi = E;
            for (int e = lane; e < E; e += 64) if (sc[e] > best || (sc[e] == best && e < bi)) { best = sc[e]; bi = e; }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const float ob = __shfl_xor(best, o, 64); const int oi = __shfl_xor(bi, o, 64);
                if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
            }
            if (bi >= E) bi = E - 1;                        // (logits that are not numbers compare false everywhere: the index still has to be an expert's)
            if (lane == 0) {
                const float sv = softmax ? expf(best - zmax) / zsum : sigmoid_f(best);
                sel[t * top + k] = bi; score[t * top + k] = sv; chosen += sv; sc[bi] = -INFINITY;
            }
        }
        __syncthreads();
    }
    if (softmax && threadIdx.x == 0) for (int k = 0; k < top; ++k) score[t * top + k] /= chosen + 1e-20f;
}

// One workgroup: counts per expert, offsets, and a place for every (token, choice) among its expert's rows.  order[place] = token * top + choice;
// place_of[token * top + choice] = place.  Which place inside its expert a row gets is left to the atomics: a row's result does not depend on it.
__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t *__restrict__ sel, int n, int E, int pad, int nblocks, int32_t *__restrict__ off,
                                                         int32_t *__restrict__ order, int32_t *__restrict__ place_of, int32_t *__restrict__ row_w) {
    extern __shared__ int32_t cnt[];                    // [E + 1] counts, then running offsets
    for (int e = threadIdx.x; e <= E; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += 1024) atomicAdd(&cnt[sel[i]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {                             // an expert's rows start at a multiple of pad; row_w names the expert of every block of pad rows
        int run = 0;
        for (int e = 0; e < E; ++e) {
            const int c = cnt[e], padded = (c + pad - 1) / pad * pad;
            cnt[e] = run; off[e] = run;
            if (row_w) for (int bk = run / pad; bk < (run + padded) / pad && bk < nblocks; ++bk) row_w[bk] = e;
            run += padded;
        }
        off[E] = run;
        if (row_w) for (int bk = run / pad; bk < nblocks; ++bk) row_w[bk] = 0;      // (blocks behind the last expert: any matrix, their rows are nobody's)
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += 1024) { const int place = atomicAdd(&cnt[sel[i]], 1); order[place] = i; place_of[i] = place; }
}

// xs[place_of[i]] = h[i / top] * score[i] (the expert's input, in the order of the grouped rows)
template <class OT>
__global__ __launch_bounds__(256) void moe_gather_kernel(const OT *__restrict__ h, int64_t ldh, int W, int top, const int32_t *__restrict__ place_of, const float *__restrict__ score,
                                                         OT *__restrict__ xs) {
    const int64_t i = blockIdx.x, t = i / top;
    const float sc = score[i];
    OT *dst = xs + (int64_t)place_of[i] * W;
    for (int c = threadIdx.x; c < W; c += 256) st_f(dst, c, ld_f(h, t * ldh + c) * sc);
}

// out[t] = sum_k y[place_of[t * top + k]] (+ shared[t]) in the operand type
template <class OT>
__global__ __launch_bounds__(256) void moe_combine_kernel(const OT *__restrict__ y, const int32_t *__restrict__ place_of, int top, const OT *__restrict__ shared, int W,
                                                          OT *__restrict__ out, const float *__restrict__ score, const float *__restrict__ shared_gate, int64_t gate_ld) {
    const int64_t t = blockIdx.x;
    const float sg = (shared && shared_gate) ? sigmoid_f(shared_gate[t * gate_ld]) : 1.f;
    for (int c = threadIdx.x; c < W; c += 256) {
        float v = shared ? ld_f(shared, t * W + c) * sg : 0.f;
        for (int k = 0; k < top; ++k) v += ld_f(y, (int64_t)place_of[t * top + k] * W + c) * (score ? score[t * top + k] : 1.f);
        st_f(out, t * W + c, v);
    }
}

// ------------------------------------------------------------------------------------------------ end of a layer
// Per row: (1) the token input's last step: x += y / rms(y) * wn for the projected rows y (side_y); (2) X_(i+1) = x goes to its
// place among the kept streams and x becomes sum_j mix[j] X_j over the nx kept streams (X_0 the embedding output ... X_(nx-1) this layer's); (3) with wnext the next layer's
// first norm (in groups) of the new x goes to out.  Each part is optional (null pointers).  The row lives in LDS.
template <class OT>
__global__ __launch_bounds__(256) void layer_tail_kernel(LayerTailArgs p) {
    extern __shared__ float sm[];                       // [W] x, [W] y
    __shared__ float red[4];
    const int64_t t = blockIdx.x; const int W = p.W, lane = threadIdx.x & 63;
    float *xs = sm, *ys = sm + W;
    float *xr = p.x + t * W;
    for (int c = threadIdx.x; c < W; c += 256) xs[c] = xr[c];
    __syncthreads();
    if (p.side_y) {
        const OT *sy = (const OT *)p.side_y + t * W;
        float ss = 0.f;
        for (int c = threadIdx.x; c < W; c += 256) { const float y = ld_f(sy, c); ys[c] = y; ss += y * y; }
        ss = block_sum256(ss, red);
        const float inv = 1.0f / sqrtf(ss / (float)W + p.eps);
        for (int c = threadIdx.x; c < W; c += 256) xs[c] += ys[c] * inv * p.side_norm[c];
        __syncthreads();
    }
    if (p.kept) {
        float *mine = p.kept + ((int64_t)(p.nx - 1) * p.kept_rows + t) * W;
        const float wl = p.mix[p.nx - 1];
        for (int c = threadIdx.x; c < W; c += 256) {
            const float v = xs[c];
            mine[c] = v;
            float acc = 0.f;
            for (int jx = 0; jx < p.nx - 1; ++jx) acc = fmaf(p.mix[jx], p.kept[((int64_t)jx * p.kept_rows + t) * W + c], acc);
            xs[c] = fmaf(wl, v, acc);
        }
        __syncthreads();
    }
    for (int c = threadIdx.x; c < W; c += 256) xr[c] = xs[c];
    if (p.wnext) {
        const int n = W / p.groups;
        OT *o = (OT *)p.out + t * W;
        for (int g = threadIdx.x >> 6; g < p.groups; g += 4) {
            float ss = 0.f;
            for (int c = lane; c < n; c += 64) { const float v = xs[g * n + c]; ss += v * v; }
            const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)n + p.eps);
            for (int c = lane; c < n; c += 64) st_f(o, g * n + c, xs[g * n + c] * inv * p.wnext[g * n + c]);
        }
    }
}

// g[t][d] = gelu_tanh(z[t][d]) * E[ids[t]][ecol + d] (the token input between its two projections)
template <class OT>
__global__ __launch_bounds__(256) void side_gate_kernel(const OT *__restrict__ z, const int64_t *__restrict__ ids, const OT *__restrict__ E, int64_t lde, int ecol, int dim,
                                                        int64_t n, OT *__restrict__ g) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int64_t t = idx / dim; const int d = (int)(idx - t * dim);
    st_f(g, idx, gelu_tanh_f(ld_f(z, idx)) * ld_f(E, ids[t] * lde + ecol + d));
}

// y[t][c] *= sigmoid(g[t][c])
template <class OT>
__global__ __launch_bounds__(256) void sigmoid_gate_kernel(OT *__restrict__ y, int64_t ldy, const OT *__restrict__ g, int64_t ldg, int64_t T, int64_t N) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= T * N) return;
    const int64_t t = idx / N, c = idx - t * N;
    st_f(y, t * ldy + c, ld_f(y, t * ldy + c) * sigmoid_f(ld_f(g, t * ldg + c)));
}

// the same for 16-bit rows, 8 numbers per thread (N and both strides multiples of 8, 16-byte aligned rows)
__global__ __launch_bounds__(256) void sigmoid_gate8_kernel(bf16_t *__restrict__ y, int64_t ldy, const bf16_t *__restrict__ g, int64_t ldg, int64_t T, int64_t N8) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= T * N8) return;
    const int64_t t = idx / N8, c = (idx - t * N8) * 8;
    uint4 yv = *reinterpret_cast<const uint4 *>(y + t * ldy + c);
    const uint4 gv = *reinterpret_cast<const uint4 *>(g + t * ldg + c);
    bf16_t *ye = reinterpret_cast<bf16_t *>(&yv); const bf16_t *ge = reinterpret_cast<const bf16_t *>(&gv);
#pragma unroll
    for (int k = 0; k < 8; ++k) st_f(ye, k, ld_f(ye, k) * sigmoid_f(ld_f(ge, k)));
    *reinterpret_cast<uint4 *>(y + t * ldy + c) = yv;
}

template <class ET>
__global__ __launch_bounds__(256) void embed_keep_kernel(const ET *__restrict__ E, const int64_t *__restrict__ ids, int W, float *__restrict__ x, float *__restrict__ kept) {
    const int64_t t = blockIdx.x, id = ids[t];
    for (int c = threadIdx.x; c < W; c += 256) { const float v = ld_f(E, id * W + c); x[t * W + c] = v; if (kept) kept[t * W + c] = v; }
}

}  // namespace

static const size_t kMaxLds = 160 * 1024 - 2048;

int prepare_blocks() {
    NVR_HIP_CHECK(hipFuncSetAttribute((const void *)layer_tail_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    NVR_HIP_CHECK(hipFuncSetAttribute((const void *)layer_tail_kernel<bf16_t>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    return 0;
}

int embed_keep(const void *E, bool bf16, const int64_t *ids, int64_t T, int64_t W, float *x, float *kept, hipStream_t s) {
    if (T == 0) return 0;
    if (bf16) embed_keep_kernel<bf16_t><<<dim3((unsigned)T), dim3(256), 0, s>>>((const bf16_t *)E, ids, (int)W, x, kept);
    else embed_keep_kernel<float><<<dim3((unsigned)T), dim3(256), 0, s>>>((const float *)E, ids, (int)W, x, kept);
    return launched("embed_keep");
}

int group_norm(const GroupNormArgs &a, bool bf16, hipStream_t s) {
    if (a.rows_n == 0) return 0;
    if (a.groups < 1 || a.W % a.groups) return nvr::fail(NVR_ERR_INVALID_ARG, "group_norm: %ld columns in %d groups", (long)a.W, a.groups);
    if (a.out_plain && (a.w2 || !a.xres)) return nvr::fail(NVR_ERR_INVALID_ARG, "group_norm: a plain copy leaves only with the residual sum, instead of the next norm");
    const dim3 grid((unsigned)a.rows_n), blk(256);
    const int W = (int)a.W;
    if (a.xres) {                                        // operand-type rows joining the f32 stream
        if (bf16) group_norm_kernel<bf16_t, bf16_t, true><<<grid, blk, 0, s>>>((const bf16_t *)a.in, a.ldi, nullptr, W, a.groups, a.eps, a.w, a.xres, a.w2, a.out_plain ? 1 : 0, (bf16_t *)a.out, a.ldo);
        else group_norm_kernel<float, float, true><<<grid, blk, 0, s>>>((const float *)a.in, a.ldi, nullptr, W, a.groups, a.eps, a.w, a.xres, a.w2, a.out_plain ? 1 : 0, (float *)a.out, a.ldo);
    } else if (a.in_f32) {
        if (bf16) group_norm_kernel<float, bf16_t, false><<<grid, blk, 0, s>>>((const float *)a.in, a.ldi, a.rows, W, a.groups, a.eps, a.w, nullptr, nullptr, 0, (bf16_t *)a.out, a.ldo);
        else group_norm_kernel<float, float, false><<<grid, blk, 0, s>>>((const float *)a.in, a.ldi, a.rows, W, a.groups, a.eps, a.w, nullptr, nullptr, 0, (float *)a.out, a.ldo);
    } else {
        if (bf16) group_norm_kernel<bf16_t, bf16_t, false><<<grid, blk, 0, s>>>((const bf16_t *)a.in, a.ldi, a.rows, W, a.groups, a.eps, a.w, nullptr, nullptr, 0, (bf16_t *)a.out, a.ldo);
        else group_norm_kernel<float, float, false><<<grid, blk, 0, s>>>((const float *)a.in, a.ldi, a.rows, W, a.groups, a.eps, a.w, nullptr, nullptr, 0, (float *)a.out, a.ldo);
    }
    return launched("group_norm");
}

int latent_store(const void *proj, int64_t ld, int64_t col, const Batch &b, int64_t rank, int64_t rot, float eps, const float *w, const float *freq, void *pages, void *rows,
                 bool bf16, hipStream_t s) {
    if (b.T == 0) return 0;
    if (rot % 2) return nvr::fail(NVR_ERR_INVALID_ARG, "latent_store: %ld rotated coordinates", (long)rot);
    if (bf16) latent_store_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(64), 0, s>>>((const bf16_t *)proj, ld, col, b, (int)rank, (int)rot, eps, w, freq, (bf16_t *)pages, (bf16_t *)rows);
    else latent_store_kernel<float><<<dim3((unsigned)b.T), dim3(64), 0, s>>>((const float *)proj, ld, col, b, (int)rank, (int)rot, eps, w, freq, (float *)pages, (float *)rows);
    return launched("latent_store");
}

int rotate_heads(const void *q, int64_t ldq, int64_t qstride, int64_t qcol, const Batch &b, int64_t H, int64_t rot, const float *freq, void *out, int64_t ldo, int64_t ostride,
                 int64_t ocol, bool bf16, hipStream_t s) {
    if (b.T == 0 || rot == 0) return 0;
    if (rot % 2) return nvr::fail(NVR_ERR_INVALID_ARG, "rotate_heads: %ld rotated coordinates", (long)rot);
    if (bf16) rotate_heads_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(256), 0, s>>>((const bf16_t *)q, ldq, (int)qstride, (int)qcol, b, (int)H, (int)rot, freq, (bf16_t *)out, ldo, (int)ostride, (int)ocol);
    else rotate_heads_kernel<float><<<dim3((unsigned)b.T), dim3(256), 0, s>>>((const float *)q, ldq, (int)qstride, (int)qcol, b, (int)H, (int)rot, freq, (float *)out, ldo, (int)ostride, (int)ocol);
    return launched("rotate_heads");
}

static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

int head_linear(const HeadLinearArgs &a, bool bf16, hipStream_t s) {
    if (a.T == 0 || a.N == 0 || a.H == 0) return 0;
    if (bf16 && a.K % 8 == 0 && a.lda % 8 == 0 && a.ha % 8 == 0 && aligned16(a.a) && aligned16(a.w)) {
        if (a.T >= 128) head_linear_mfma128_kernel<<<dim3((unsigned)((a.N + 127) / 128), (unsigned)((a.T + 127) / 128), (unsigned)a.H), dim3(256), 0, s>>>(a);
        else if (a.T <= 16) head_linear_ksplit_kernel<<<dim3((unsigned)((a.N + 63) / 64), (unsigned)((a.T + 15) / 16), (unsigned)a.H), dim3(256), 0, s>>>(a);
        else head_linear_mfma_kernel<4><<<dim3((unsigned)((a.N + 63) / 64), (unsigned)((a.T + 63) / 64), (unsigned)a.H), dim3(256), 0, s>>>(a);
        return launched("head_linear");
    }
    const dim3 grid((unsigned)((a.N + 63) / 64), (unsigned)((a.T + 63) / 64), (unsigned)a.H);
    if (bf16) head_linear_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(a);
    else head_linear_kernel<float><<<grid, dim3(256), 0, s>>>(a);
    return launched("head_linear");
}

int grouped_linear(const GroupedLinearArgs &a, bool bf16, hipStream_t s) {
    if (a.max_rows == 0 || a.N == 0 || a.groups == 0) return 0;
    if (bf16 && a.K % 8 == 0 && a.lda % 8 == 0 && aligned16(a.a) && aligned16(a.w)) {
        if (a.max_rows >= 96 * a.groups) grouped_linear_mfma128_kernel<<<dim3((unsigned)((a.N + 127) / 128), (unsigned)(a.max_rows / 128 + a.groups)), dim3(256), 0, s>>>(a);
        else if (a.max_rows <= 16 * a.groups) grouped_linear_ksplit_kernel<<<dim3((unsigned)((a.N + 63) / 64), (unsigned)(a.max_rows / 16 + a.groups)), dim3(256), 0, s>>>(a);
        else grouped_linear_mfma_kernel<4><<<dim3((unsigned)((a.N + 63) / 64), (unsigned)(a.max_rows / 64 + a.groups)), dim3(256), 0, s>>>(a);
        return launched("grouped_linear");
    }
    const dim3 grid((unsigned)((a.N + 63) / 64), (unsigned)(a.max_rows / 64 + a.groups));
    if (bf16) grouped_linear_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(a);
    else grouped_linear_kernel<float><<<grid, dim3(256), 0, s>>>(a);
    return launched("grouped_linear");
}

int poly_norm(const void *z, int64_t ldz, int64_t T, int64_t F, float eps, const float *coef, void *out, int64_t ldo, bool bf16, hipStream_t s) {
    if (T == 0) return 0;
    if (bf16) poly_norm_kernel<bf16_t><<<dim3((unsigned)T), dim3(256), 0, s>>>((const bf16_t *)z, ldz, (int)F, eps, coef, (bf16_t *)out, ldo);
    else poly_norm_kernel<float><<<dim3((unsigned)T), dim3(256), 0, s>>>((const float *)z, ldz, (int)F, eps, coef, (float *)out, ldo);
    return launched("poly_norm");
}

int silu_mul(const void *gu, int64_t T, int64_t F, void *out, int64_t ldo, bool bf16, hipStream_t s) {
    if (T * F == 0) return 0;
    const dim3 grid((unsigned)((T * F + 255) / 256));
    if (bf16) silu_mul_kernel<bf16_t><<<grid, dim3(256), 0, s>>>((const bf16_t *)gu, T, F, (bf16_t *)out, ldo);
    else silu_mul_kernel<float><<<grid, dim3(256), 0, s>>>((const float *)gu, T, F, (float *)out, ldo);
    return launched("silu_mul");
}

int moe_route(const void *h, int64_t ldh, int64_t T, int64_t W, const float *wr, int64_t E, int64_t top, int32_t *sel, float *score, int32_t *off, int32_t *order,
              int32_t *place_of, int64_t pad, int32_t *row_w, int64_t nblocks, bool bf16, hipStream_t s, bool softmax, int64_t extra, float *extra_out,
              const float *logits, int64_t ldl) {
    if (T == 0) return 0;
    if (extra < 0 || (extra > 0 && !extra_out)) return nvr::fail(NVR_ERR_INVALID_ARG, "moe_route: %ld further rows without a place for them", (long)extra);
    if (top < 1 || top > E) return nvr::fail(NVR_ERR_INVALID_ARG, "moe_route: %ld of %ld experts", (long)top, (long)E);
    if ((size_t)(E + 1) * 4 > 60000) return nvr::fail(NVR_ERR_UNSUPPORTED, "moe_route: %ld experts", (long)E);
    if (bf16) moe_route_kernel<bf16_t><<<dim3((unsigned)T), dim3(256), (size_t)(E + extra) * 4, s>>>((const bf16_t *)h, ldh, (int)W, wr, (int)E, (int)top, sel, score, softmax ? 1 : 0, (int)extra, extra_out, logits, ldl);
    else moe_route_kernel<float><<<dim3((unsigned)T), dim3(256), (size_t)(E + extra) * 4, s>>>((const float *)h, ldh, (int)W, wr, (int)E, (int)top, sel, score, softmax ? 1 : 0, (int)extra, extra_out, logits, ldl);
    if (int rc = launched("moe_route")) return rc;
    if (pad < 1) return nvr::fail(NVR_ERR_INVALID_ARG, "moe_route: rows padded to %ld", (long)pad);
    moe_group_kernel<<<dim3(1), dim3(1024), (size_t)(E + 1) * 4, s>>>(sel, (int)(T * top), (int)E, (int)pad, (int)nblocks, off, order, place_of, row_w);
    return launched("moe_group");
}

int moe_gather(const void *h, int64_t ldh, int64_t T, int64_t W, int64_t top, const int32_t *place_of, const float *score, void *xs, bool bf16, hipStream_t s) {
    if (T * top == 0) return 0;
    if (bf16) moe_gather_kernel<bf16_t><<<dim3((unsigned)(T * top)), dim3(256), 0, s>>>((const bf16_t *)h, ldh, (int)W, (int)top, place_of, score, (bf16_t *)xs);
    else moe_gather_kernel<float><<<dim3((unsigned)(T * top)), dim3(256), 0, s>>>((const float *)h, ldh, (int)W, (int)top, place_of, score, (float *)xs);
    return launched("moe_gather");
}

int moe_combine(const void *y, const int32_t *place_of, int64_t T, int64_t top, const void *shared, int64_t W, void *out, bool bf16, hipStream_t s,
                const float *score, const float *shared_gate, int64_t gate_ld) {
    if (T == 0) return 0;
    if (bf16) moe_combine_kernel<bf16_t><<<dim3((unsigned)T), dim3(256), 0, s>>>((const bf16_t *)y, place_of, (int)top, (const bf16_t *)shared, (int)W, (bf16_t *)out, score, shared_gate, gate_ld);
    else moe_combine_kernel<float><<<dim3((unsigned)T), dim3(256), 0, s>>>((const float *)y, place_of, (int)top, (const float *)shared, (int)W, (float *)out, score, shared_gate, gate_ld);
    return launched("moe_combine");
}

int sigmoid_gate(void *y, int64_t ldy, const void *g, int64_t ldg, int64_t T, int64_t N, bool bf16, hipStream_t s) {
    if (T * N == 0) return 0;
    if (bf16 && N % 8 == 0 && ldy % 8 == 0 && ldg % 8 == 0 && (((uintptr_t)y | (uintptr_t)g) & 15) == 0) {
        sigmoid_gate8_kernel<<<dim3((unsigned)((T * (N / 8) + 255) / 256)), dim3(256), 0, s>>>((bf16_t *)y, ldy, (const bf16_t *)g, ldg, T, N / 8);
        return launched("sigmoid_gate");
    }
    const dim3 grid((unsigned)((T * N + 255) / 256));
    if (bf16) sigmoid_gate_kernel<bf16_t><<<grid, dim3(256), 0, s>>>((bf16_t *)y, ldy, (const bf16_t *)g, ldg, T, N);
    else sigmoid_gate_kernel<float><<<grid, dim3(256), 0, s>>>((float *)y, ldy, (const float *)g, ldg, T, N);
    return launched("sigmoid_gate");
}

int side_gate(const void *z, const int64_t *ids, const void *E, int64_t lde, int64_t ecol, int64_t dim, int64_t T, void *g, bool bf16, hipStream_t s) {
    if (T * dim == 0) return 0;
    const dim3 grid((unsigned)((T * dim + 255) / 256));
    if (bf16) side_gate_kernel<bf16_t><<<grid, dim3(256), 0, s>>>((const bf16_t *)z, ids, (const bf16_t *)E, lde, (int)ecol, (int)dim, T * dim, (bf16_t *)g);
    else side_gate_kernel<float><<<grid, dim3(256), 0, s>>>((const float *)z, ids, (const float *)E, lde, (int)ecol, (int)dim, T * dim, (float *)g);
    return launched("side_gate");
}

int layer_tail(const LayerTailArgs &a, bool bf16, hipStream_t s) {
    if (a.T == 0) return 0;
    const size_t lds = (size_t)2 * a.W * 4;
    if (lds > kMaxLds) return nvr::fail(NVR_ERR_UNSUPPORTED, "layer_tail: rows of %d numbers do not fit LDS", a.W);
    if (a.wnext && (a.groups < 1 || a.W % a.groups)) return nvr::fail(NVR_ERR_INVALID_ARG, "layer_tail: %d columns in %d groups", a.W, a.groups);
    if (bf16) layer_tail_kernel<bf16_t><<<dim3((unsigned)a.T), dim3(256), lds, s>>>(a);
    else layer_tail_kernel<float><<<dim3((unsigned)a.T), dim3(256), lds, s>>>(a);
    return launched("layer_tail");
}

}}  // namespace nvr::kl
