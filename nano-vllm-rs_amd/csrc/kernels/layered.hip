// layered.hip — kernels of layer-list models (kernels/layered.h): f32 residual stream, scalar-gain RMS norm + causal convolution in front
// of each sublayer, attention with distance penalty and sink, retention with f32 state, clamped gated feed-forward.  wave64, gfx950.
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

__device__ __forceinline__ void st4_f(float *p, int64_t i, const float (&v)[4]) { *reinterpret_cast<float4 *>(p + i) = float4{v[0], v[1], v[2], v[3]}; }
__device__ __forceinline__ void st4_f(bf16_t *p, int64_t i, const float (&v)[4]) {       // i a multiple of 4: one 8-byte store
    bf16_t h[4];
#pragma unroll
    for (int y = 0; y < 4; ++y) st_f(h, y, v[y]);
    *reinterpret_cast<uint2 *>(p + i) = uint2{(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
}

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
// sum over a workgroup of NT threads (NT a multiple of 64, <= 1024); red: NT/64 floats of LDS; every thread gets the sum
template <int NT>
__device__ __forceinline__ float block_sum(float v, float *red) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NT / 64; ++i) t += red[i];
    return t;
}
template <int NT>
__device__ __forceinline__ float block_max(float v, float *red) {
    v = wave_max(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = red[0];
#pragma unroll
    for (int i = 1; i < NT / 64; ++i) t = fmaxf(t, red[i]);
    return t;
}

int launched(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return nvr::fail(NVR_ERR_HIP, "%s launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

// ------------------------------------------------------------------------------------------------ embedding
template <class ET>
__global__ __launch_bounds__(256) void embed_scale_kernel(const ET *__restrict__ E, const int64_t *__restrict__ ids, int W, float scale, float *__restrict__ x) {
    const int64_t t = blockIdx.x;
    const int64_t id = ids[t];
    for (int c = threadIdx.x; c < W; c += 256) x[t * W + c] = ld_f(E, id * W + c) * scale;
}

// ------------------------------------------------------------------------------------------------ norm + causal convolution
// One workgroup per row.  u[d] (d = 0: this row, d: the row d positions back) is brought into LDS: rows of this step are normalised here, rows before the
// chunk come from the history, rows before position 0 are zero.
template <class OT>
__global__ __launch_bounds__(256) void norm_canon_kernel(const float *__restrict__ x, Batch b, int W, float eps, int taps, float g1, const float *__restrict__ w1,
                                                         OT *__restrict__ out1, float g2, const float *__restrict__ w2, OT *__restrict__ out2,
                                                         float *__restrict__ hist, int64_t slots) {
    extern __shared__ float u[];                        // [taps][W]
    __shared__ float red[4];
    const int t = blockIdx.x, sq = b.row_seq[t];
    const int c0 = b.cu[sq], i = t - c0, n = b.cu[sq + 1] - c0, st = b.start[sq];
    const int64_t slot = b.slot[sq]; const int par = b.par[sq];
    const int hrows = taps - 1;
    const float *hin = hist + ((int64_t)par * slots + slot) * hrows * W;
    float *hout = hist + ((int64_t)(par ^ 1) * slots + slot) * hrows * W;
    for (int d = 0; d < taps; ++d) {
        float *ud = u + (int64_t)d * W;
        if (i - d >= 0) {
            const float *xr = x + (int64_t)(t - d) * W;
            float ss = 0.f;
            for (int c = threadIdx.x; c < W; c += 256) { const float v = xr[c]; ud[c] = v; ss += v * v; }
            ss = block_sum<256>(ss, red);
            const float r = 1.0f / sqrtf(ss / (float)W + eps);
            for (int c = threadIdx.x; c < W; c += 256) ud[c] *= r;
        } else if (st + i - d >= 0) {
            const float *hr = hin + (int64_t)(hrows + (i - d)) * W;           // history row e holds position start - hrows + e
            for (int c = threadIdx.x; c < W; c += 256) ud[c] = hr[c];
        } else {
            for (int c = threadIdx.x; c < W; c += 256) ud[c] = 0.f;
        }
    }
    __syncthreads();
    for (int c = threadIdx.x; c < W; c += 256) {
        const float u0 = u[c];
        float a1 = 0.f, a2 = 0.f;
        for (int j = 0; j < taps; ++j) {
            const float uv = u[(int64_t)(taps - 1 - j) * W + c];
            a1 += w1[(int64_t)c * taps + j] * (g1 * uv);
            if (out2) a2 += w2[(int64_t)c * taps + j] * (g2 * uv);
        }
        st_f(out1, (int64_t)t * W + c, g1 * u0 + a1);
        if (out2) st_f(out2, (int64_t)t * W + c, g2 * u0 + a2);
    }
    if (i == n - 1)                                     // the chunk's last row leaves the history of the next step: positions end - hrows .. end - 1
        for (int d = 0; d < hrows; ++d)
            for (int c = threadIdx.x; c < W; c += 256) hout[(int64_t)(hrows - 1 - d) * W + c] = u[(int64_t)d * W + c];
}

// The same for widths that are multiples of 4 and up to 8 taps, RB rows per workgroup and nothing staged in LDS: the waves first reduce the rows the group
// needs (its own and the taps-1 before them) to 1 / rms each, then every thread walks its columns four at a time and gathers, per output row, the taps inputs
// from the step's rows (L1 / L2 hits: a row is read by up to taps neighbours), the slot's history, or zero.
template <class OT, int RB>
__global__ __launch_bounds__(256) void norm_canon_rows_kernel(const float *__restrict__ x, Batch b, int W, float eps, int taps, float g1, const float *__restrict__ w1,
                                                              OT *__restrict__ out1, float g2, const float *__restrict__ w2, OT *__restrict__ out2,
                                                              float *__restrict__ hist, int64_t slots) {
    __shared__ float rinv[RB + 8];
    __shared__ int rs_i[RB], rs_n[RB], rs_st[RB], rs_par[RB]; __shared__ int64_t rs_slot[RB];
    const int t0 = blockIdx.x * RB, hrows = taps - 1;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int k = wave; k < RB + hrows; k += 4) {
        const int gr = t0 - hrows + k;
        if (gr < 0 || gr >= b.T) continue;
        const float4 *xr = reinterpret_cast<const float4 *>(x + (int64_t)gr * W);
        float ss = 0.f;
        for (int c = lane; c < (W >> 2); c += 64) { const float4 v = xr[c]; ss += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w); }
        ss = wave_sum(ss);
        if (lane == 0) rinv[k] = 1.0f / sqrtf(ss / (float)W + eps);
    }
    if (threadIdx.x < RB && t0 + threadIdx.x < b.T) {
        const int t = t0 + threadIdx.x, sq = b.row_seq[t], c0 = b.cu[sq];
        rs_i[threadIdx.x] = t - c0; rs_n[threadIdx.x] = b.cu[sq + 1] - c0; rs_st[threadIdx.x] = b.start[sq]; rs_par[threadIdx.x] = b.par[sq]; rs_slot[threadIdx.x] = b.slot[sq];
    }
    __syncthreads();
    for (int c4 = threadIdx.x * 4; c4 < W; c4 += 1024) {
        float wa[4][8], wb[4][8];
#pragma unroll
        for (int y = 0; y < 4; ++y)
#pragma unroll
            for (int j = 0; j < 8; ++j) { wa[y][j] = j < taps ? w1[(int64_t)(c4 + y) * taps + j] : 0.f; wb[y][j] = (out2 && j < taps) ? w2[(int64_t)(c4 + y) * taps + j] : 0.f; }
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            const int t = t0 + r;
            if (t >= b.T) break;
            const int i = rs_i[r], st = rs_st[r];
            const float *hin = hist + ((int64_t)rs_par[r] * slots + rs_slot[r]) * hrows * W;
            float *hout = hist + ((int64_t)(rs_par[r] ^ 1) * slots + rs_slot[r]) * hrows * W;
            const bool last = i == rs_n[r] - 1;
            float a1[4] = {0.f, 0.f, 0.f, 0.f}, a2[4] = {0.f, 0.f, 0.f, 0.f}, u0[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 8; ++j) {                       // tap j weighs the row taps - 1 - j back
                if (j >= taps) break;
                const int d = taps - 1 - j;
                float4 u = float4{0.f, 0.f, 0.f, 0.f};
                if (i - d >= 0) {
                    const float ri = rinv[r + hrows - d];
                    u = *reinterpret_cast<const float4 *>(x + (int64_t)(t - d) * W + c4);
                    u.x *= ri; u.y *= ri; u.z *= ri; u.w *= ri;
                } else if (st + i - d >= 0) u = *reinterpret_cast<const float4 *>(hin + (int64_t)(hrows + (i - d)) * W + c4);
                const float uu[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int y = 0; y < 4; ++y) {
                    a1[y] += wa[y][j] * (g1 * uu[y]); a2[y] += wb[y][j] * (g2 * uu[y]);
                    if (d == 0) u0[y] = uu[y];
                }
                if (last && d < hrows) *reinterpret_cast<float4 *>(hout + (int64_t)(hrows - 1 - d) * W + c4) = u;
            }
            float o1[4], o2[4];
#pragma unroll
            for (int y = 0; y < 4; ++y) { o1[y] = g1 * u0[y] + a1[y]; o2[y] = g2 * u0[y] + a2[y]; }
            st4_f(out1, (int64_t)t * W + c4, o1);
            if (out2) st4_f(out2, (int64_t)t * W + c4, o2);
        }
    }
}

// ------------------------------------------------------------------------------------------------ K / V rows into the paged caches
template <class CT>
__global__ __launch_bounds__(256) void kv_store_kernel(const CT *__restrict__ proj, int64_t ld, int64_t kcol, int64_t vcol, Batch b, int G, int D, int Dv,
                                                       CT *__restrict__ kc, CT *__restrict__ vc, int grouped) {
    const int t = blockIdx.x, sq = b.row_seq[t];
    const int p = b.start[sq] + (t - b.cu[sq]);
    const int blk = b.block_tables[(int64_t)sq * b.max_blocks + p / b.block_size];
    const int64_t row = (int64_t)blk * b.block_size + p % b.block_size;
    const CT *pr = proj + (int64_t)t * ld;
    for (int c = threadIdx.x; c < G * D; c += 256) kc[row * G * D + c] = pr[kcol + c];
    if (!grouped) { for (int c = threadIdx.x; c < G * Dv; c += 256) vc[row * G * Dv + c] = pr[vcol + c]; return; }
    const int jj = p % b.block_size;                    // value pages in groups of 8 keys per column: [block][block_size / 8][G][Dv][8]
    const int64_t grp = ((int64_t)blk * (b.block_size >> 3) + (jj >> 3)) * G * Dv;
    for (int c = threadIdx.x; c < G * Dv; c += 256) vc[(grp + c) * 8 + (jj & 7)] = pr[vcol + c];
}

// ------------------------------------------------------------------------------------------------ attention with distance penalty and sink
// General form (any D, Dv, context that fits LDS): one workgroup per (row, head); scores of all visible keys in LDS, then the weighted sum of values.
template <class CT>
__global__ __launch_bounds__(256) void sink_attn_rows_kernel(SinkAttnArgs a, Batch b) {
    extern __shared__ float sm[];                       // [D] q, [ctx] scores, [256] partial outputs
    __shared__ float red[4];
    const int t = blockIdx.x, h = blockIdx.y, sq = b.row_seq[t];
    const int i = b.start[sq] + (t - b.cu[sq]), ctx = i + 1;
    const int kvh = h / (a.H / a.G);
    float *qs = sm, *sc = sm + a.D;
    const CT *q = (const CT *)a.q + (int64_t)t * a.ldq + (int64_t)h * a.D;
    for (int d = threadIdx.x; d < a.D; d += 256) qs[d] = ld_f(q, d);
    __syncthreads();
    const CT *kc = (const CT *)a.kc; const CT *vc = (const CT *)a.vc;
    const int32_t *bt = b.block_tables + (int64_t)sq * b.max_blocks;
    const float r1 = a.r1 ? a.r1[h] : 0.f, r2 = a.r2 ? a.r2[h] : 0.f, slope = a.slope ? a.slope[h] : 0.f;
    int j0 = a.window > 0 ? max(0, ctx - a.window) : 0;            // first visible key; the score buffer holds the keys j0 .. ctx - 1
    if (a.chunk > 0) j0 = max(j0, i / a.chunk * a.chunk);          // (chunks count from position 0 of the sequence)
    const bool gate = a.gate_bias != nullptr;                      // weights sigmoid(score + bias), not normalised
    const float gb = gate ? a.gate_bias[h] : 0.f;
    sc -= j0;
    float mx = a.sink ? a.sink[h] : -INFINITY;
    for (int j = j0 + threadIdx.x; j < ctx; j += 256) {
        const int64_t row = (int64_t)bt[j / b.block_size] * b.block_size + j % b.block_size;
        const int64_t base = (row * a.G + kvh) * a.D;
        float dot = 0.f;
        for (int d = 0; d < a.D; ++d) dot += qs[d] * ld_f(kc, base + d);
        float s = dot * a.scale;
        if (a.r1) s -= r1 * log1pf(r2 * (float)(i - j));
        if (a.slope) s -= slope * (float)(i - j);
        if (a.softcap > 0.f) s = a.softcap * tanhf(s / a.softcap);
        if (gate) s = 1.0f / (1.0f + expf(-(s + gb)));
        sc[j] = s;
        mx = fmaxf(mx, s);
    }
    float inv = 1.0f;
    if (gate) __syncthreads();                          // (publishes the weights)
    else {
    mx = block_max<256>(mx, red);
    float sum = 0.f;
    for (int j = j0 + threadIdx.x; j < ctx; j += 256) { const float e = expf(sc[j] - mx); sc[j] = e; sum += e; }
    sum = block_sum<256>(sum, red);                     // (its barriers also publish the weights)
    if (a.sink) sum += expf(a.sink[h] - mx);
    inv = 1.0f / sum;
    }
    // values: column c by lanes, keys split over the 256 / CW groups
    float *part = sc + ctx;                             // (behind the last score)
    const int64_t vld = a.vld ? a.vld : a.Dv;           // (values inside the key rows: the latent of latent attention)
    for (int cb = 0; cb < a.Dv; cb += 64) {
        const int c = cb + (threadIdx.x & 63), grp = threadIdx.x >> 6;
        float acc = 0.f;
        if (c < a.Dv)
            for (int j = j0 + grp; j < ctx; j += 4) {
                const int64_t row = (int64_t)bt[j / b.block_size] * b.block_size + j % b.block_size;
                acc += sc[j] * ld_f(vc, (row * a.G + kvh) * vld + c);
            }
        part[threadIdx.x] = acc;
        __syncthreads();
        if (grp == 0 && c < a.Dv) {
            const float o = (part[threadIdx.x] + part[threadIdx.x + 64]) + (part[threadIdx.x + 128] + part[threadIdx.x + 192]);
            st_f((CT *)a.out, (int64_t)t * a.ldo + (int64_t)h * a.Dv + c, o * inv);
        }
        __syncthreads();
    }
}

// Matrix-core form (bf16 operands; D and Dv multiples of 32 / 16 up to the size class C).  A workgroup owns one tile — up to 64 / g consecutive
// positions of one sequence times the g = H / G query heads of one key/value head, 16 rows per wave — and walks the keys in tiles of 64 through LDS:
// S = Q K^T on v_mfma_f32_16x16x32_bf16, penalty / mask / online softmax in f32 on the accumulator layout (lane: key column, four rows), P rounded
// to bf16 through LDS into the A layout, O += P V.  The value pages are stored in groups of 8 keys per column ([.][G][Dv][8]), so that a B fragment
// of P V (8 consecutive keys of one column) is one 16-byte read.  The distance penalty comes from a table per head (penalty_table_kernel), everything
// in the base-2 domain (v_exp_f32 is 2^x).  The next tile's keys and values are requested before the current tile's arithmetic and land in LDS after
// it.  The sink starts the running maximum and counts 1 in the running sum.  nsplit > 1: workgroup z takes every nsplit-th tile of keys and leaves
// (o, m, l) partials for sink_attn_merge_kernel.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr float kLog2e = 1.4426950408889634f;

__global__ __launch_bounds__(256) void penalty_table_kernel(const float *__restrict__ r1, const float *__restrict__ r2, int H, int n, float *__restrict__ tab) {
    const int d = blockIdx.x * 256 + threadIdx.x, h = blockIdx.y;
    if (d < n) tab[(int64_t)h * n + d] = (r2 ? r1[h] * log1pf(r2[h] * (float)d) : r1[h] * (float)d) * kLog2e;      // (r2 null: linear in the distance)
}

// GATE: no softmax — the weight of a visible key is sigmoid(capped score + bias of the head), the tiles' products are summed as they are (a split's partial carries
// m = 0 and the first split l = 1, so that the merge adds the partials up).  chunk > 0 (both forms): a row sees the keys from its chunk's first position on.
template <int C, bool GATE = false>
__global__ __launch_bounds__(256, 2) void sink_attn_mfma_kernel(SinkAttnArgs a, Batch b, const AttnTile *__restrict__ tiles, int nsplit, float *__restrict__ part_o,
                                                             float *__restrict__ part_ml) {
    constexpr int KT = 64, KS = C + 8, VS = KT + 8, VG = C + 1, NCH = C / 32;   // NCH: 16-byte pieces of a K (or V) tile per thread
    extern __shared__ char smem[];
    bf16_t *Ks = (bf16_t *)smem;                        // [KT][KS] keys x dims
    bf16_t *Vg = Ks + KT * KS;                          // [8 key groups][VG columns][8 keys]
    bf16_t *Ps = Vg + 8 * VG * 8;                       // [4][16][VS] one wave's weights
    float *pen = (float *)(Ps + 64 * VS);               // [g][128] penalties of the distances this key tile can have
    const int tile = blockIdx.x, kvh = blockIdx.y, z = blockIdx.z;
    const int sq = tiles[tile].seq, lr0 = tiles[tile].row0;
    const int c0 = b.cu[sq], n = b.cu[sq + 1] - c0, st = b.start[sq];
    const int g = a.H / a.G, PW = 64 / g;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lm = lane & 15, lq = lane >> 4;
    const int D = a.D, Dv = a.Dv, d32 = D >> 5, dv16 = Dv >> 4;
    const int npos = min(PW, n - lr0);                  // positions of this tile
    const bool wave_on = wave * 16 < npos * g;
    const bf16_t *kc = (const bf16_t *)a.kc, *vc = (const bf16_t *)a.vc;
    const int32_t *bt = b.block_tables + (int64_t)sq * b.max_blocks;
    const int bs = b.block_size, bs8 = bs >> 3;
    const float scale2 = a.scale * kLog2e;

    bf16x8 qf[C / 32];
    {
        const int r = wave * 16 + lm, pi = min(r / g, npos - 1), hg = r % g;
        const bf16_t *q = (const bf16_t *)a.q + (int64_t)(c0 + lr0 + pi) * a.ldq + (int64_t)(kvh * g + hg) * D + lq * 8;
#pragma unroll
        for (int ks = 0; ks < C / 32; ++ks) if (ks < d32) qf[ks] = *reinterpret_cast<const bf16x8 *>(q + ks * 32);
    }
    int pos[4], hgi[4], cs[4]; float m[4], l[4], gb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = wave * 16 + lq * 4 + i, h = kvh * g + r % g;
        pos[i] = st + lr0 + r / g; hgi[i] = r % g;
        cs[i] = a.chunk > 0 ? pos[i] / a.chunk * a.chunk : 0;      // first key of the row's chunk
        const bool sink_here = a.sink && z == 0;
        m[i] = GATE ? 0.f : sink_here ? a.sink[h] * kLog2e : -INFINITY;
        l[i] = ((GATE || sink_here) && z == 0 && lm == 0) ? 1.f : 0.f;
        gb[i] = GATE ? a.gate_bias[h] : 0.f;
    }
    f32x4 acc[C / 16];
#pragma unroll
    for (int t = 0; t < C / 16; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int p0 = st + lr0;                            // first position of the tile
    const int nkeys = p0 + npos;                        // keys the tile's last position sees
    const int ntl = (nkeys + KT - 1) / KT;
    int kt0 = a.window > 0 ? max(p0 - a.window + 1, 0) / KT : 0;            // first key tile the tile's first position can see
    if (a.chunk > 0) kt0 = max(kt0, p0 / a.chunk * a.chunk / KT);
    const int kch = D >> 3;
    uint4 kreg[NCH], vreg[NCH];
    // a thread's pieces: key skey, 16-byte pieces sch, sch + 4, ... of its row; key group vkg, columns vcl, vcl + 32, ... (one block-table lookup each per tile)
    const int skey = threadIdx.x >> 2, sch = threadIdx.x & 3, vkg = threadIdx.x >> 5, vcl = threadIdx.x & 31;
    auto request = [&](int k0) {                        // pieces of the key tile at k0 -> registers
        const int jk = k0 + skey, jv = k0 + vkg * 8;
        const int bk = jk < nkeys ? jk / bs : 0, bv = jv < nkeys ? jv / bs : 0;
        const bf16_t *kr = kc + (((int64_t)bt[bk] * bs + (jk - bk * bs)) * a.G + kvh) * D;
        const bf16_t *vr = vc + (((int64_t)bt[bv] * bs8 + ((jv - bv * bs) >> 3)) * a.G + kvh) * Dv * 8;
        const bf16_t *vrow = vc + (((int64_t)bt[bk] * bs + (jk - bk * bs)) * a.G + kvh) * (a.vld ? a.vld : (int64_t)Dv);      // row-major pages: the key's own row
#pragma unroll
        for (int x = 0; x < NCH; ++x) {
            kreg[x] = uint4{0, 0, 0, 0}; vreg[x] = uint4{0, 0, 0, 0};
            if (jk < nkeys && sch + 4 * x < kch) kreg[x] = *reinterpret_cast<const uint4 *>(kr + (sch + 4 * x) * 8);
            if (a.v_grouped) { if (jv < nkeys && vcl + 32 * x < Dv) vreg[x] = *reinterpret_cast<const uint4 *>(vr + (vcl + 32 * x) * 8); }
            else if (jk < nkeys && sch + 4 * x < (Dv >> 3)) vreg[x] = *reinterpret_cast<const uint4 *>(vrow + (sch + 4 * x) * 8);
        }
    };
    if (kt0 + z < ntl) request((kt0 + z) * KT);
    for (int kt = kt0 + z; kt < ntl; kt += nsplit) {
        const int k0 = kt * KT;
        const int dmin = max(p0 - (k0 + KT - 1), 0);    // smallest distance a visible key of this tile can have
        __syncthreads();
#pragma unroll
        for (int x = 0; x < NCH; ++x) {
            if (sch + 4 * x < kch) *reinterpret_cast<uint4 *>(Ks + skey * KS + (sch + 4 * x) * 8) = kreg[x];
            if (a.v_grouped) { if (vcl + 32 * x < Dv) *reinterpret_cast<uint4 *>(Vg + (vkg * VG + vcl + 32 * x) * 8) = vreg[x]; }
            else if (sch + 4 * x < (Dv >> 3)) {                                  // 8 columns of one key: into the key-group layout, element by element
                const bf16_t *e = reinterpret_cast<const bf16_t *>(&vreg[x]);
#pragma unroll
                for (int y = 0; y < 8; ++y) Vg[((skey >> 3) * VG + (sch + 4 * x) * 8 + y) * 8 + (skey & 7)] = e[y];
            }
        }
        if (a.pen)
            for (int idx = threadIdx.x; idx < g * 128; idx += 256) {
                const int hg = idx >> 7, d = dmin + (idx & 127);
                pen[idx] = d < a.pen_n ? a.pen[(int64_t)(kvh * g + hg) * a.pen_n + d] : 0.f;
            }
        __syncthreads();
        if (kt + nsplit < ntl) request((kt + nsplit) * KT);
        if (wave_on) {
            f32x4 s[4];
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
                s[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < C / 32; ++ks)
                    if (ks < d32) {
                        const bf16x8 kf = *reinterpret_cast<const bf16x8 *>(Ks + (nt * 16 + lm) * KS + ks * 32 + lq * 8);
                        s[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], kf, s[nt], 0, 0, 0);
                    }
            }
            if (GATE) {
                const float c2 = a.softcap > 0.f ? 2.0f * kLog2e / a.softcap : 0.f;
#pragma unroll
                for (int nt = 0; nt < 4; ++nt) {
                    const int j = k0 + nt * 16 + lm;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float v = s[nt][i] * a.scale;
                        if (a.softcap > 0.f) v = a.softcap * (1.0f - 2.0f / (exp2f(v * c2) + 1.0f));      // cap * tanh(v / cap)
                        const float p = (j > pos[i] || j < cs[i]) ? 0.f : 1.0f / (1.0f + exp2f(-kLog2e * (v + gb[i])));
                        const __bf16 pb = (__bf16)p;
                        Ps[(wave * 16 + lq * 4 + i) * VS + nt * 16 + lm] = __builtin_bit_cast(bf16_t, pb);
                    }
                }
            } else {
            float mx[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
                const int j = k0 + nt * 16 + lm;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int dist = pos[i] - j;
                    float v = s[nt][i] * scale2;
                    if (a.pen) v -= pen[(hgi[i] << 7) + min(max(dist - dmin, 0), 127)];
                    v = (dist < 0 || (a.window > 0 && dist >= a.window) || j < cs[i]) ? -INFINITY : v;
                    s[nt][i] = v;
                    mx[i] = fmaxf(mx[i], v);
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma unroll
                for (int o = 1; o < 16; o <<= 1) mx[i] = fmaxf(mx[i], __shfl_xor(mx[i], o, 64));
                const float mn = fmaxf(m[i], mx[i]);
                const float alpha = (m[i] == -INFINITY) ? 0.f : exp2f(m[i] - mn);
                const float ms = (mn == -INFINITY) ? 0.f : mn;
                m[i] = mn;
                float rs = 0.f;
#pragma unroll
                for (int nt = 0; nt < 4; ++nt) {
                    const float p = exp2f(s[nt][i] - ms);                // (a masked key: 2^-inf = 0)
                    rs += p;
                    const __bf16 pb = (__bf16)p;
                    Ps[(wave * 16 + lq * 4 + i) * VS + nt * 16 + lm] = __builtin_bit_cast(bf16_t, pb);
                }
                l[i] = l[i] * alpha + rs;
#pragma unroll
                for (int t = 0; t < C / 16; ++t) acc[t][i] *= alpha;
            }
            }
            __builtin_amdgcn_wave_barrier();                // (the weights are read back by this wave only: LDS serves a wave's requests in order)
#pragma unroll
            for (int k2 = 0; k2 < KT / 32; ++k2) {
                const bf16x8 pf = *reinterpret_cast<const bf16x8 *>(Ps + (wave * 16 + lm) * VS + k2 * 32 + lq * 8);
#pragma unroll
                for (int t = 0; t < C / 16; ++t)
                    if (t < dv16) {
                        const bf16x8 vf = *reinterpret_cast<const bf16x8 *>(Vg + ((k2 * 4 + lq) * VG + t * 16 + lm) * 8);
                        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf, acc[t], 0, 0, 0);
                    }
            }
        }
    }
    if (!wave_on) return;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) l[i] += __shfl_xor(l[i], o, 64);
        const int r = wave * 16 + lq * 4 + i, pi = r / g, hg = r % g;
        if (pi >= npos) continue;
        if (nsplit == 1) {
            const float inv = 1.0f / l[i];
            bf16_t *o = (bf16_t *)a.out + (int64_t)(c0 + lr0 + pi) * a.ldo + (int64_t)(kvh * g + hg) * Dv;
#pragma unroll
            for (int t = 0; t < C / 16; ++t) if (t < dv16) st_f(o, t * 16 + lm, acc[t][i] * inv);
        } else {
            const int64_t pr = (((int64_t)tile * a.G + kvh) * nsplit + z) * 64 + r;
#pragma unroll
            for (int t = 0; t < C / 16; ++t) if (t < dv16) part_o[pr * Dv + t * 16 + lm] = acc[t][i];
            if (lm == 0) { part_ml[pr * 2] = m[i]; part_ml[pr * 2 + 1] = l[i]; }
        }
    }
}

// one wave per (tile, key/value head, row): out = sum_z o_z 2^(m_z - m) / sum_z l_z 2^(m_z - m)
__global__ __launch_bounds__(64) void sink_attn_merge_kernel(SinkAttnArgs a, Batch b, const AttnTile *__restrict__ tiles, int nsplit, const float *__restrict__ part_o,
                                                             const float *__restrict__ part_ml) {
    const int tile = blockIdx.x, kvh = blockIdx.y, r = blockIdx.z;
    const int sq = tiles[tile].seq, lr0 = tiles[tile].row0;
    const int c0 = b.cu[sq], n = b.cu[sq + 1] - c0;
    const int g = a.H / a.G, PW = 64 / g, npos = min(PW, n - lr0);
    const int pi = r / g, hg = r % g;
    if (pi >= npos) return;
    const int64_t base = ((int64_t)tile * a.G + kvh) * nsplit;
    float m = -INFINITY;
    for (int z = 0; z < nsplit; ++z) m = fmaxf(m, part_ml[((base + z) * 64 + r) * 2]);
    float l = 0.f;
    for (int z = 0; z < nsplit; ++z) { const float mz = part_ml[((base + z) * 64 + r) * 2]; if (mz != -INFINITY) l += part_ml[((base + z) * 64 + r) * 2 + 1] * exp2f(mz - m); }
    bf16_t *o = (bf16_t *)a.out + (int64_t)(c0 + lr0 + pi) * a.ldo + (int64_t)(kvh * g + hg) * a.Dv;
    for (int c = threadIdx.x; c < a.Dv; c += 64) {
        float acc = 0.f;
        for (int z = 0; z < nsplit; ++z) { const float mz = part_ml[((base + z) * 64 + r) * 2]; if (mz != -INFINITY) acc += part_o[((base + z) * 64 + r) * a.Dv + c] * exp2f(mz - m); }
        st_f(o, c, acc / l);
    }
}

// ------------------------------------------------------------------------------------------------ retention, token by token
// One workgroup per (sequence, head, block of 32 value columns): thread (c, part) keeps rows part, part + 8, ... of column c of the state in registers.
// log(sigmoid(z)) without overflow
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <int RMAX, class PT, int MODE>
__global__ __launch_bounds__(256) void retention_seq_kernel(RetentionArgs a, Batch b) {
    constexpr bool GATED = MODE != 0, PRE = MODE == 2;      // PRE: the output is read before the update, the current token enters it through the bonus
    __shared__ float qs[2][512], ks[2][512], red[8][32];
    __shared__ float as[GATED ? 2 : 1][GATED ? 512 : 1];
    const int sq = blockIdx.x, h = blockIdx.y, cb = blockIdx.z * 32;
    const int c = cb + (threadIdx.x & 31), part = threadIdx.x >> 5;
    const int r0 = b.cu[sq], n = b.cu[sq + 1] - r0, st = b.start[sq];
    const int D = a.D, Dv = a.Dv, half = a.rot_dims / 2;
    const int hq = a.qk_share > 1 ? h / a.qk_share : h;    // the head whose q and k this head reads
    const bool tok = !GATED && a.tok_gate != nullptr;     // (keep, take) per token and head instead of decay[h]
    const float dec = (GATED || tok) ? 0.f : a.decay[h];
    const int Dr = Dv - a.v_ones;                          // value columns that proj holds; the rest are ones
    float *S = a.state + (((int64_t)b.slot[sq] * a.H + h) * D) * Dv;
    const bool live = c < Dv;
    float s[RMAX], ub[PRE ? RMAX : 1];
#pragma unroll
    for (int r = 0; r < RMAX; ++r) { const int d = part + r * 8; s[r] = (st > 0 && live && d < D) ? S[(int64_t)d * Dv + c] : 0.f; if (PRE) ub[PRE ? r : 0] = d < D ? a.bonus[(int64_t)h * D + d] : 0.f; }
    for (int i = 0; i < n; ++i) {
        const int t = r0 + i, buf = i & 1;
        const float keep = tok ? a.tok_gate[((int64_t)t * a.H + h) * 2] : dec, take = tok ? a.tok_gate[((int64_t)t * a.H + h) * 2 + 1] : 1.f;
        const PT *pr = (const PT *)a.proj + (int64_t)t * a.ld;
        const PT *q = pr + a.qcol + (int64_t)hq * D, *k = pr + a.kcol + (int64_t)hq * D;
        for (int d = threadIdx.x; d < D; d += 256) {
            float qv = ld_f(q, d), kv = ld_f(k, d);
            if (d < a.rot_dims) {
                const int fi = d < half ? d : d - half;
                const int64_t p = st + i;
                const float cs = a.cos_t[p * half + fi], sn = a.sin_t[p * half + fi];
                if (d < half) { qv = qv * cs - ld_f(q, d + half) * sn; kv = kv * cs - ld_f(k, d + half) * sn; }
                else { qv = qv * cs + ld_f(q, d - half) * sn; kv = kv * cs + ld_f(k, d - half) * sn; }
            }
            if (GATED) {
                qv *= a.qscale;
                const float z = ld_f((const PT *)a.az, (int64_t)t * a.ldz + (int64_t)h * D + d) + a.abias[(int64_t)h * D + d];
                as[buf][d] = a.decay_exp ? expf(-expf(z)) : expf(log_sigmoid(z) * a.inv_tau);
            }
            if (tok) { qv *= a.qscale; kv *= take; }
            qs[buf][d] = qv; ks[buf][d] = kv * a.kscale;
        }
        __syncthreads();
        const float v = live ? (c < Dr ? ld_f(pr, a.vcol + (int64_t)h * Dr + c) : 1.f) : 0.f;
        float o = 0.f;
#pragma unroll
        for (int r = 0; r < RMAX; ++r) {
            const int d = part + r * 8;
            if (d < D) {
                if (PRE) { const float kv = ks[buf][d] * v; o += (s[r] + ub[PRE ? r : 0] * kv) * qs[buf][d]; s[r] = as[buf][d] * s[r] + kv; }
                else { s[r] = (GATED ? as[buf][d] : keep) * s[r] + ks[buf][d] * v; o += s[r] * qs[buf][d]; }
            }
        }
        red[part][threadIdx.x & 31] = o;
        __syncthreads();
        if (part == 0 && live) {
            float tot = 0.f;
#pragma unroll
            for (int p2 = 0; p2 < 8; ++p2) tot += red[p2][threadIdx.x];
            a.o[(int64_t)t * a.H * Dv + (int64_t)h * Dv + c] = tot;
        }
        // (red is rewritten two barriers later: after the next token's first barrier every reader of this token's sums has passed)
    }
    if (live)
#pragma unroll
        for (int r = 0; r < RMAX; ++r) { const int d = part + r * 8; if (d < D) S[(int64_t)d * Dv + c] = s[r]; }
}

// The same recurrence, 16 tokens per barrier (key size up to 256): a pass brings the rotated q, scaled rotated k and v of its tokens into LDS (cosines
// and sines from the position table), every thread then walks the tokens with its rows of the state in registers and leaves its partial outputs in LDS; one
// barrier later they are summed over the 8 row groups.  Token order and arithmetic per token are those of the token-by-token kernel: the result does not depend
// on where a prompt is cut.  Thread (c, part) owns rows part * RMAX .. part * RMAX + RMAX - 1 of column c.
// GATED: the decay is per token and key channel, sigmoid(z + bias)^(1/tau) with z from rows of the operand type, and q is scaled by qscale (gated linear attention).
template <int RMAX, class PT, int MODE>
__global__ __launch_bounds__(256) void retention_block_kernel(RetentionArgs a, Batch b) {
    constexpr bool GATED = MODE != 0, PRE = MODE == 2;
    constexpr int TB = 16;
    extern __shared__ float rsm[];
    const int D = a.D, Dv = a.Dv, half = a.rot_dims / 2;
    const int hq = a.qk_share > 1 ? (int)blockIdx.y / a.qk_share : (int)blockIdx.y;
    float *qs = rsm, *ks = qs + TB * D, *vs = ks + TB * D, *partial = vs + TB * 32;      // [TB][D], [TB][D], [TB][32], [TB][8][32]
    float *as = partial + TB * 8 * 32;                                                    // GATED: [TB][D] decays; token-gated: [TB] keep, [TB] take
    const int sq = blockIdx.x, h = blockIdx.y, cb = blockIdx.z * 32;
    const int cl = threadIdx.x & 31, c = cb + cl, part = threadIdx.x >> 5;
    const int r0 = b.cu[sq], n = b.cu[sq + 1] - r0, st = b.start[sq];
    const bool tok = !GATED && a.tok_gate != nullptr;
    const float dec = (GATED || tok) ? 0.f : a.decay[h];
    const int Dr = Dv - a.v_ones;
    // One column of ones (the gated running sum n of the keys) is not given a column block of its own: the launch covers the Dr columns that proj holds, and the
    // first block also walks n, one row per thread (row part * RMAX + cl of the threads with cl < RMAX), and sums n . q over the threads by shuffles.
    const bool fold = tok && a.v_ones == 1;
    const int Dc = fold ? Dr : Dv;                         // columns the launch's blocks cover
    float *S = a.state + (((int64_t)b.slot[sq] * a.H + h) * D) * Dv;
    const bool live = c < Dc;
    float s[RMAX], ub[PRE ? RMAX : 1];
#pragma unroll
    for (int r = 0; r < RMAX; ++r) { const int d = part * RMAX + r; s[r] = (st > 0 && live && d < D) ? S[(int64_t)d * Dv + c] : 0.f; if (PRE) ub[PRE ? r : 0] = d < D ? a.bonus[(int64_t)h * D + d] : 0.f; }
    const int dn = part * RMAX + cl;
    const bool nblock = fold && blockIdx.z == 0, nown = nblock && cl < RMAX && dn < D;
    float sn = (nown && st > 0) ? S[(int64_t)dn * Dv + Dv - 1] : 0.f;
    float *partial_n = as + 2 * TB;                        // [TB][8]
    for (int i0 = 0; i0 < n; i0 += TB) {
        const int nb = min(TB, n - i0);
        __syncthreads();
        if (tok) {
            if (threadIdx.x < 2 * nb) as[(threadIdx.x & 1) * TB + (threadIdx.x >> 1)] = a.tok_gate[((int64_t)(r0 + i0 + (threadIdx.x >> 1)) * a.H + h) * 2 + (threadIdx.x & 1)];
            __syncthreads();
        }
        const int dsh = (D & (D - 1)) == 0 ? 31 - __clz(D) : -1;
        // fully rotated bf16 heads: a thread takes 8 coordinates of the lower half and their partners of the upper half as 16-byte loads
        const bool fast = !GATED && !tok && sizeof(PT) == 2 && a.rot_dims == D && (half & 7) == 0 && (a.ld & 7) == 0 && ((a.qcol | a.kcol) & 7) == 0 && ((uintptr_t)a.proj & 15) == 0;
        if (fast) {
            const int cpt = half >> 3;                                   // 8-coordinate pieces of a half
            for (int idx = threadIdx.x; idx < nb * cpt; idx += 256) {
                const int i = idx / cpt, d0 = (idx - i * cpt) << 3;
                const bf16_t *pr = (const bf16_t *)a.proj + (int64_t)(r0 + i0 + i) * a.ld;
                const bf16_t *q = pr + a.qcol + (int64_t)hq * D + d0, *k = pr + a.kcol + (int64_t)hq * D + d0;
                const uint4 ql = *reinterpret_cast<const uint4 *>(q), qh = *reinterpret_cast<const uint4 *>(q + half);
                const uint4 kl = *reinterpret_cast<const uint4 *>(k), kh = *reinterpret_cast<const uint4 *>(k + half);
                const int64_t p = st + i0 + i;
                const float *cp = a.cos_t + p * half + d0, *sp = a.sin_t + p * half + d0;
                const bf16_t *qle = reinterpret_cast<const bf16_t *>(&ql), *qhe = reinterpret_cast<const bf16_t *>(&qh);
                const bf16_t *kle = reinterpret_cast<const bf16_t *>(&kl), *khe = reinterpret_cast<const bf16_t *>(&kh);
#pragma unroll
                for (int y = 0; y < 8; ++y) {
                    const float cs = cp[y], sn = sp[y];
                    const float qu = ld_f(qle, y), qv = ld_f(qhe, y), ku = ld_f(kle, y), kv = ld_f(khe, y);
                    qs[i * D + d0 + y] = qu * cs - qv * sn; qs[i * D + half + d0 + y] = qv * cs + qu * sn;
                    ks[i * D + d0 + y] = (ku * cs - kv * sn) * a.kscale; ks[i * D + half + d0 + y] = (kv * cs + ku * sn) * a.kscale;
                }
            }
        } else if (GATED && sizeof(PT) == 2 && a.rot_dims == 0 && (D & 7) == 0 && (a.ld & 7) == 0 && ((a.qcol | a.kcol | a.ldz) & 7) == 0 && (((uintptr_t)a.proj | (uintptr_t)a.az) & 15) == 0) {
            // gated, 16-bit rows: a thread takes 8 consecutive channels of one token as 16-byte loads; the decay (1 + e^-z)^(-1/tau) through the hardware's
            // base-2 exponential and logarithm (z -> -inf gives 0, no overflow on the way)
            const int cpt = D >> 3;
            for (int idx = threadIdx.x; idx < nb * cpt; idx += 256) {
                const int i = idx / cpt, d0 = (idx - i * cpt) << 3;
                const bf16_t *pr = (const bf16_t *)a.proj + (int64_t)(r0 + i0 + i) * a.ld;
                const uint4 qv = *reinterpret_cast<const uint4 *>(pr + a.qcol + (int64_t)hq * D + d0), kv = *reinterpret_cast<const uint4 *>(pr + a.kcol + (int64_t)hq * D + d0);
                const uint4 zv = *reinterpret_cast<const uint4 *>((const bf16_t *)a.az + (int64_t)(r0 + i0 + i) * a.ldz + (int64_t)h * D + d0);
                const bf16_t *qe = reinterpret_cast<const bf16_t *>(&qv), *ke = reinterpret_cast<const bf16_t *>(&kv), *ze = reinterpret_cast<const bf16_t *>(&zv);
                const float *bp = a.abias + (int64_t)h * D + d0;
#pragma unroll
                for (int y = 0; y < 8; ++y) {
                    qs[i * D + d0 + y] = ld_f(qe, y) * a.qscale; ks[i * D + d0 + y] = ld_f(ke, y) * a.kscale;
                    as[i * D + d0 + y] = a.decay_exp ? exp2f(-kLog2e * exp2f(kLog2e * (ld_f(ze, y) + bp[y]))) : exp2f(-a.inv_tau * __log2f(1.0f + exp2f(-kLog2e * (ld_f(ze, y) + bp[y]))));
                }
            }
        } else if (tok && sizeof(PT) == 2 && a.rot_dims == 0 && (D & 7) == 0 && (a.ld & 7) == 0 && ((a.qcol | a.kcol) & 7) == 0 && ((uintptr_t)a.proj & 15) == 0) {
            // token-gated, 16-bit rows: 8 consecutive channels of one token as 16-byte loads; the token's input gate rides on its key
            const int cpt = D >> 3;
            for (int idx = threadIdx.x; idx < nb * cpt; idx += 256) {
                const int i = idx / cpt, d0 = (idx - i * cpt) << 3;
                const bf16_t *pr = (const bf16_t *)a.proj + (int64_t)(r0 + i0 + i) * a.ld;
                const uint4 qv = *reinterpret_cast<const uint4 *>(pr + a.qcol + (int64_t)hq * D + d0), kv = *reinterpret_cast<const uint4 *>(pr + a.kcol + (int64_t)hq * D + d0);
                const bf16_t *qe = reinterpret_cast<const bf16_t *>(&qv), *ke = reinterpret_cast<const bf16_t *>(&kv);
                const float take = as[TB + i];
#pragma unroll
                for (int y = 0; y < 8; ++y) { qs[i * D + d0 + y] = ld_f(qe, y) * a.qscale; ks[i * D + d0 + y] = ld_f(ke, y) * take * a.kscale; }
            }
        } else
        for (int idx = threadIdx.x; idx < nb * D; idx += 256) {
            const int i = dsh >= 0 ? idx >> dsh : idx / D, d = idx - i * D;
            const PT *pr = (const PT *)a.proj + (int64_t)(r0 + i0 + i) * a.ld;
            const PT *q = pr + a.qcol + (int64_t)hq * D, *k = pr + a.kcol + (int64_t)hq * D;
            float qv = ld_f(q, d), kv = ld_f(k, d);
            if (d < a.rot_dims) {
                const int fi = d < half ? d : d - half;
                const int64_t p = st + i0 + i;
                const float cs = a.cos_t[p * half + fi], sn = a.sin_t[p * half + fi];
                if (d < half) { qv = qv * cs - ld_f(q, d + half) * sn; kv = kv * cs - ld_f(k, d + half) * sn; }
                else { qv = qv * cs + ld_f(q, d - half) * sn; kv = kv * cs + ld_f(k, d - half) * sn; }
            }
            if (GATED) {
                qv *= a.qscale;
                const float z = ld_f((const PT *)a.az, (int64_t)(r0 + i0 + i) * a.ldz + (int64_t)h * D + d) + a.abias[(int64_t)h * D + d];
                as[idx] = a.decay_exp ? expf(-expf(z)) : expf(log_sigmoid(z) * a.inv_tau);
            }
            if (tok) { qv *= a.qscale; kv *= as[TB + i]; }
            qs[idx] = qv; ks[idx] = kv * a.kscale;
        }
        for (int idx = threadIdx.x; idx < nb * 32; idx += 256) {
            const int i = idx >> 5, cc = cb + (idx & 31);
            vs[idx] = cc < Dc ? (cc < Dr ? ld_f((const PT *)a.proj + (int64_t)(r0 + i0 + i) * a.ld, a.vcol + (int64_t)h * Dr + cc) : 1.f) : 0.f;
        }
        __syncthreads();
        for (int i = 0; i < nb; ++i) {
            const float v = vs[i * 32 + cl];
            const float *kr = ks + i * D + part * RMAX, *qr = qs + i * D + part * RMAX;
            float o = 0.f;
            if (GATED) {
                const float *ar = as + i * D + part * RMAX;
                if (D == 8 * RMAX) {
                    float kk[RMAX], qq[RMAX], aa[RMAX];
#pragma unroll
                    for (int r = 0; r < RMAX; r += 4) {
                        *reinterpret_cast<float4 *>(kk + r) = *reinterpret_cast<const float4 *>(kr + r);
                        *reinterpret_cast<float4 *>(qq + r) = *reinterpret_cast<const float4 *>(qr + r);
                        *reinterpret_cast<float4 *>(aa + r) = *reinterpret_cast<const float4 *>(ar + r);
                    }
#pragma unroll
                    for (int r = 0; r < RMAX; ++r) {
                        if (PRE) { const float kv = kk[r] * v; o += (s[r] + ub[PRE ? r : 0] * kv) * qq[r]; s[r] = aa[r] * s[r] + kv; }
                        else { s[r] = aa[r] * s[r] + kk[r] * v; o += s[r] * qq[r]; }
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < RMAX; ++r)
                        if (part * RMAX + r < D) {
                            if (PRE) { const float kv = kr[r] * v; o += (s[r] + ub[PRE ? r : 0] * kv) * qr[r]; s[r] = ar[r] * s[r] + kv; }
                            else { s[r] = ar[r] * s[r] + kr[r] * v; o += s[r] * qr[r]; }
                        }
                }
            } else if (D == 8 * RMAX) {
                const float dd = tok ? as[i] : dec;
                float kk[RMAX], qq[RMAX];
#pragma unroll
                for (int r = 0; r < RMAX; r += 4) {
                    *reinterpret_cast<float4 *>(kk + r) = *reinterpret_cast<const float4 *>(kr + r);
                    *reinterpret_cast<float4 *>(qq + r) = *reinterpret_cast<const float4 *>(qr + r);
                }
#pragma unroll
                for (int r = 0; r < RMAX; ++r) { s[r] = dd * s[r] + kk[r] * v; o += s[r] * qq[r]; }
            } else {
                const float dd = tok ? as[i] : dec;
#pragma unroll
                for (int r = 0; r < RMAX; ++r)
                    if (part * RMAX + r < D) { s[r] = dd * s[r] + kr[r] * v; o += s[r] * qr[r]; }
            }
            partial[(i * 8 + part) * 32 + cl] = o;
            if (nblock) {                                   // (uniform over the workgroup)
                float on = 0.f;
                if (nown) { sn = as[i] * sn + ks[i * D + dn]; on = sn * qs[i * D + dn]; }
#pragma unroll
                for (int off = 16; off > 0; off >>= 1) on += __shfl_xor(on, off, 64);      // over the 32 lanes of the part
                if (cl == 0) partial_n[i * 8 + part] = on;
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < nb * 32; idx += 256) {
            const int i = idx >> 5, cc = cb + (idx & 31);
            float tot = 0.f;
#pragma unroll
            for (int p2 = 0; p2 < 8; ++p2) tot += partial[(i * 8 + p2) * 32 + (idx & 31)];
            if (cc < Dc) a.o[(int64_t)(r0 + i0 + i) * a.H * Dv + (int64_t)h * Dv + cc] = tot;
        }
        if (nblock && threadIdx.x < nb) {
            float tot = 0.f;
#pragma unroll
            for (int p2 = 0; p2 < 8; ++p2) tot += partial_n[threadIdx.x * 8 + p2];
            a.o[(int64_t)(r0 + i0 + threadIdx.x) * a.H * Dv + (int64_t)h * Dv + Dv - 1] = tot;
        }
    }
    if (live)
#pragma unroll
        for (int r = 0; r < RMAX; ++r) { const int d = part * RMAX + r; if (d < D) S[(int64_t)d * Dv + c] = s[r]; }
    if (nown) S[(int64_t)dn * Dv + Dv - 1] = sn;
}

template <class OT>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float *__restrict__ o, const OT *__restrict__ gate, int64_t ldg, int64_t gcol, int H, int Dv,
                                                             float eps, const float *__restrict__ w, OT *__restrict__ out, int64_t ldo, int w_heads) {
    const int64_t t = blockIdx.x; const int lane = threadIdx.x & 63;
    for (int h = threadIdx.x >> 6; h < H; h += 4) {              // a wave per head
        const float *orow = o + (t * H + h) * Dv;
        float ss = 0.f;
        for (int c = lane; c < Dv; c += 64) { const float v = orow[c]; ss += v * v; }
        ss = wave_sum(ss);
        const float r = 1.0f / sqrtf(ss / (float)Dv + eps);
        for (int c = lane; c < Dv; c += 64) {
            const float g = ld_f(gate, t * ldg + gcol + (int64_t)h * Dv + c);
            st_f(out, t * ldo + (int64_t)h * Dv + c, orow[c] * r * (w ? w[w_heads ? h * Dv + c : c] : 1.0f) * (g / (1.0f + expf(-g))));
        }
    }
}

template <class OT>
__global__ __launch_bounds__(256) void clamped_glu_kernel(const OT *__restrict__ gu, int64_t T, int64_t F, float limit, float alpha, OT *__restrict__ out, int64_t ldo) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= T * F) return;
    const int64_t t = idx / F, c = idx - t * F;
    const float g = fminf(ld_f(gu, t * 2 * F + c), limit);
    const float u = fminf(fmaxf(ld_f(gu, t * 2 * F + F + c), -limit), limit);
    st_f(out, t * ldo + c, g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
}

// the same, 8 bf16 elements (16 bytes) per thread: F and ldo multiples of 8
__global__ __launch_bounds__(256) void clamped_glu8_kernel(const bf16_t *__restrict__ gu, int64_t T, int64_t F, float limit, float alpha, bf16_t *__restrict__ out, int64_t ldo) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x, f8 = F >> 3;
    if (idx >= T * f8) return;
    const int64_t t = idx / f8, c = (idx - t * f8) << 3;
    const uint4 gv = *reinterpret_cast<const uint4 *>(gu + t * 2 * F + c), uv = *reinterpret_cast<const uint4 *>(gu + t * 2 * F + F + c);
    const bf16_t *ge = reinterpret_cast<const bf16_t *>(&gv), *ue = reinterpret_cast<const bf16_t *>(&uv);
    uint4 ov; bf16_t *oe = reinterpret_cast<bf16_t *>(&ov);
#pragma unroll
    for (int x = 0; x < 8; ++x) {
        const float g = fminf(ld_f(ge, x), limit), u = fminf(fmaxf(ld_f(ue, x), -limit), limit);
        st_f(oe, x, g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
    }
    *reinterpret_cast<uint4 *>(out + t * ldo + c) = ov;
}

template <class YT>
__global__ __launch_bounds__(256) void axpy_kernel(float *__restrict__ x, const YT *__restrict__ y, float m, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) x[i] += m * ld_f(y, i);
}

template <class OT>
__global__ __launch_bounds__(256) void norm_rows_kernel(const float *__restrict__ x, const int32_t *__restrict__ rows, int W, float eps, float g, OT *__restrict__ out) {
    __shared__ float red[4];
    const int64_t r = blockIdx.x;
    const float *xr = x + (int64_t)rows[r] * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) { const float v = xr[c]; ss += v * v; }
    ss = block_sum<256>(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += 256) st_f(out, r * W + c, xr[c] * rs * g);
}

template <class ET, class YT>
__global__ __launch_bounds__(256) void gemm_any_kernel(const ET *__restrict__ a, int64_t lda, const ET *__restrict__ w, int T, int K, int N, YT *__restrict__ y) {
    __shared__ float as[16][17], ws[16][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int t = blockIdx.y * 16 + ty, nn = blockIdx.x * 16 + tx;
    float acc = 0.f;
    for (int k0 = 0; k0 < K; k0 += 16) {
        const int ka = k0 + tx;
        as[ty][tx] = (t < T && ka < K) ? ld_f(a, (int64_t)t * lda + ka) : 0.f;
        const int wn = blockIdx.x * 16 + ty;
        ws[ty][tx] = (wn < N && ka < K) ? ld_f(w, (int64_t)wn * K + ka) : 0.f;
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) acc += as[ty][kk] * ws[tx][kk];
        __syncthreads();
    }
    if (t < T && nn < N) st_f(y, (int64_t)t * N + nn, acc);
}

}  // namespace

static const size_t kMaxLds = 160 * 1024 - 2048;

int prepare() {
    NVR_HIP_CHECK(hipFuncSetAttribute((const void *)sink_attn_rows_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    NVR_HIP_CHECK(hipFuncSetAttribute((const void *)sink_attn_rows_kernel<bf16_t>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    NVR_HIP_CHECK(hipFuncSetAttribute((const void *)sink_attn_mfma_kernel<64>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    NVR_HIP_CHECK(hipFuncSetAttribute((const void *)sink_attn_mfma_kernel<128>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    NVR_HIP_CHECK(hipFuncSetAttribute((const void *)sink_attn_mfma_kernel<256>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    NVR_HIP_CHECK(hipFuncSetAttribute((const void *)sink_attn_mfma_kernel<64, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    NVR_HIP_CHECK(hipFuncSetAttribute((const void *)sink_attn_mfma_kernel<128, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    NVR_HIP_CHECK(hipFuncSetAttribute((const void *)sink_attn_mfma_kernel<256, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    NVR_HIP_CHECK(hipFuncSetAttribute((const void *)norm_canon_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    NVR_HIP_CHECK(hipFuncSetAttribute((const void *)norm_canon_kernel<bf16_t>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    return 0;
}

int embed_scale(const void *E, bool bf16, const int64_t *ids, int64_t T, int64_t W, float scale, float *x, hipStream_t s) {
    if (T == 0) return 0;
    if (bf16) embed_scale_kernel<bf16_t><<<dim3((unsigned)T), dim3(256), 0, s>>>((const bf16_t *)E, ids, (int)W, scale, x);
    else embed_scale_kernel<float><<<dim3((unsigned)T), dim3(256), 0, s>>>((const float *)E, ids, (int)W, scale, x);
    return launched("embed_scale");
}

int norm_canon(const float *x, const Batch &b, int64_t W, float eps, int taps, float g1, const float *w1, void *out1, float g2, const float *w2, void *out2,
               bool bf16, float *hist, int64_t slots, hipStream_t s) {
    if (b.T == 0) return 0;
    if (taps < 1) return nvr::fail(NVR_ERR_INVALID_ARG, "norm_canon: taps %d (at least 1)", taps);
    if (W % 4 == 0 && taps <= 8 && ((uintptr_t)x | (uintptr_t)hist) % 16 == 0) {
        // rows per workgroup: many for prompts (the convolution weights of a column are read once per workgroup), few for decode-sized steps (more workgroups)
#define NVR_NC(RB_)                                                                                                                                       \
    do {                                                                                                                                                  \
        const dim3 grid((unsigned)((b.T + RB_ - 1) / RB_));                                                                                               \
        if (bf16) norm_canon_rows_kernel<bf16_t, RB_><<<grid, dim3(256), 0, s>>>(x, b, (int)W, eps, taps, g1, w1, (bf16_t *)out1, g2, w2, (bf16_t *)out2, hist, slots); \
        else norm_canon_rows_kernel<float, RB_><<<grid, dim3(256), 0, s>>>(x, b, (int)W, eps, taps, g1, w1, (float *)out1, g2, w2, (float *)out2, hist, slots);        \
    } while (0)
        if (b.T >= 4096) NVR_NC(16); else if (b.T >= 64) NVR_NC(4); else NVR_NC(1);
#undef NVR_NC
        return launched("norm_canon");
    }
    const size_t lds = (size_t)taps * (size_t)W * 4;
    if (lds > kMaxLds) return nvr::fail(NVR_ERR_UNSUPPORTED, "norm_canon: %d taps of %ld channels do not fit LDS", taps, (long)W);
    if (bf16) norm_canon_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(256), lds, s>>>(x, b, (int)W, eps, taps, g1, w1, (bf16_t *)out1, g2, w2, (bf16_t *)out2, hist, slots);
    else norm_canon_kernel<float><<<dim3((unsigned)b.T), dim3(256), lds, s>>>(x, b, (int)W, eps, taps, g1, w1, (float *)out1, g2, w2, (float *)out2, hist, slots);
    return launched("norm_canon");
}

int kv_store(const void *proj, int64_t ld, int64_t kcol, int64_t vcol, const Batch &b, int64_t G, int64_t D, int64_t Dv, void *kc, void *vc, bool bf16,
             bool v_grouped, hipStream_t s) {
    if (v_grouped && b.block_size % 8) return nvr::fail(NVR_ERR_INVALID_ARG, "kv_store: grouped value pages need a block size that is a multiple of 8");
    if (b.T == 0) return 0;
    if (bf16) kv_store_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(256), 0, s>>>((const bf16_t *)proj, ld, kcol, vcol, b, (int)G, (int)D, (int)Dv, (bf16_t *)kc, (bf16_t *)vc, (int)v_grouped);
    else kv_store_kernel<float><<<dim3((unsigned)b.T), dim3(256), 0, s>>>((const float *)proj, ld, kcol, vcol, b, (int)G, (int)D, (int)Dv, (float *)kc, (float *)vc, (int)v_grouped);
    return launched("kv_store");
}

bool sink_attention_tiled_ok(const SinkAttnArgs &a, bool bf16, int block_size) {
    return bf16 && (block_size % 8 == 0 || !a.v_grouped) && a.G >= 1 && a.H % a.G == 0 && a.H / a.G <= 16 && a.D % 32 == 0 && a.Dv % 16 == 0 && a.D <= 256 && a.Dv <= 256 && a.ldq % 8 == 0 && a.vld % 8 == 0 && (!a.vld || !a.v_grouped) &&
           ((uintptr_t)a.q % 16) == 0 && ((uintptr_t)a.kc % 16) == 0 && ((uintptr_t)a.vc % 16) == 0;
}
size_t sink_attention_workspace_bytes(int max_workgroups) { return (size_t)max_workgroups * 64 * (256 + 2) * sizeof(float); }

int sink_attention_tiled(const SinkAttnArgs &a, const Batch &b, const AttnTile *tiles, int ntiles, int nsplit, void *workspace, size_t workspace_bytes, hipStream_t s) {
    if (ntiles == 0) return 0;
    if (!sink_attention_tiled_ok(a, true, b.block_size) || (a.v_grouped && b.block_size % 8)) return nvr::fail(NVR_ERR_UNSUPPORTED, "sink_attention_tiled: shape outside the matrix-core kernel");
    if (nsplit < 1) nsplit = 1;
    float *po = nullptr, *pml = nullptr;
    if (nsplit > 1) {
        const size_t rows = (size_t)ntiles * a.G * nsplit * 64;
        if (rows * (a.Dv + 2) * sizeof(float) > workspace_bytes) return nvr::fail(NVR_ERR_INVALID_ARG, "sink_attention_tiled: workspace too small for %d splits", nsplit);
        po = (float *)workspace; pml = po + rows * a.Dv;
    }
    const int C = std::max(a.D, a.Dv) <= 64 ? 64 : std::max(a.D, a.Dv) <= 128 ? 128 : 256;
    const size_t lds = ((size_t)64 * (C + 8) + (size_t)8 * (C + 1) * 8 + (size_t)64 * 72) * 2 + (size_t)(a.H / a.G) * 128 * 4;
    const dim3 grid((unsigned)ntiles, (unsigned)a.G, (unsigned)nsplit);
    if (a.gate_bias) {
        if (a.r1 || a.r2 || a.slope || a.sink || a.pen) return nvr::fail(NVR_ERR_INVALID_ARG, "sink_attention_tiled: gated weights take no penalty and no sink");
        if (C == 64) sink_attn_mfma_kernel<64, true><<<grid, dim3(256), lds, s>>>(a, b, tiles, nsplit, po, pml);
        else if (C == 128) sink_attn_mfma_kernel<128, true><<<grid, dim3(256), lds, s>>>(a, b, tiles, nsplit, po, pml);
        else sink_attn_mfma_kernel<256, true><<<grid, dim3(256), lds, s>>>(a, b, tiles, nsplit, po, pml);
    } else if (C == 64) sink_attn_mfma_kernel<64><<<grid, dim3(256), lds, s>>>(a, b, tiles, nsplit, po, pml);
    else if (C == 128) sink_attn_mfma_kernel<128><<<grid, dim3(256), lds, s>>>(a, b, tiles, nsplit, po, pml);
    else sink_attn_mfma_kernel<256><<<grid, dim3(256), lds, s>>>(a, b, tiles, nsplit, po, pml);
    if (int rc = launched("sink_attention_tiled")) return rc;
    if (nsplit > 1) {
        const int g = a.H / a.G, rows = std::min(64, std::max(1, std::min(64 / g, (int)b.max_rows)) * g);      // rows a tile of this step can hold
        sink_attn_merge_kernel<<<dim3((unsigned)ntiles, (unsigned)a.G, (unsigned)rows), dim3(64), 0, s>>>(a, b, tiles, nsplit, po, pml);
        return launched("sink_attention merge");
    }
    return 0;
}

int penalty_table(const float *r1, const float *r2, int64_t H, int64_t n, float *tab, hipStream_t s) {
    if (H * n == 0) return 0;
    penalty_table_kernel<<<dim3((unsigned)((n + 255) / 256), (unsigned)H), dim3(256), 0, s>>>(r1, r2, (int)H, (int)n, tab);
    return launched("penalty_table");
}
int linear_penalty_table(const float *slope, int64_t H, int64_t n, float *tab, hipStream_t s) {
    if (H * n == 0) return 0;
    penalty_table_kernel<<<dim3((unsigned)((n + 255) / 256), (unsigned)H), dim3(256), 0, s>>>(slope, nullptr, (int)H, (int)n, tab);
    return launched("linear_penalty_table");
}

int sink_attention(const SinkAttnArgs &a, const Batch &b, bool bf16, hipStream_t s) {
    if (b.T == 0) return 0;
    if (a.G < 1 || a.H % a.G) return nvr::fail(NVR_ERR_INVALID_ARG, "sink_attention: %d heads over %d key/value heads", a.H, a.G);
    if ((a.r1 || a.r2) && a.slope) return nvr::fail(NVR_ERR_INVALID_ARG, "sink_attention: a logarithmic and a linear penalty together");
    size_t keys = a.window > 0 ? (size_t)std::min(b.max_ctx, a.window) : (size_t)b.max_ctx;
    if (a.chunk > 0) keys = std::min(keys, (size_t)a.chunk);
    if (a.gate_bias && (a.r1 || a.r2 || a.slope || a.sink)) return nvr::fail(NVR_ERR_INVALID_ARG, "sink_attention: gated weights take no penalty and no sink");
    const size_t lds = ((size_t)a.D + keys + 256) * 4;
    if (lds > kMaxLds) return nvr::fail(NVR_ERR_UNSUPPORTED, "sink_attention: %zu visible keys do not fit the score buffer", keys);
    const dim3 grid((unsigned)b.T, (unsigned)a.H);
    if (bf16) sink_attn_rows_kernel<bf16_t><<<grid, dim3(256), lds, s>>>(a, b);
    else sink_attn_rows_kernel<float><<<grid, dim3(256), lds, s>>>(a, b);
    return launched("sink_attention");
}

int retention(const RetentionArgs &a, const Batch &b, bool bf16, hipStream_t s) {
    if (b.T == 0) return 0;
    if (a.D > 512) return nvr::fail(NVR_ERR_UNSUPPORTED, "retention: key size %d (at most 512)", a.D);
    if (a.rot_dims % 2 || a.rot_dims > a.D) return nvr::fail(NVR_ERR_INVALID_ARG, "retention: %d rotated coordinates of %d", a.rot_dims, a.D);
    const dim3 grid((unsigned)b.B, (unsigned)a.H, (unsigned)((a.Dv + 31) / 32));
    const int rows = (a.D + 7) / 8;
    const bool gated = a.az != nullptr;
    if (gated && !a.abias) return nvr::fail(NVR_ERR_INVALID_ARG, "retention: gated decays need their bias");
    if (gated && a.tok_gate) return nvr::fail(NVR_ERR_INVALID_ARG, "retention: decays per channel and gates per token together");
    if (a.bonus && !gated) return nvr::fail(NVR_ERR_INVALID_ARG, "retention: a bonus belongs to the gated form");
    if (a.qk_share > 1 && a.H % a.qk_share) return nvr::fail(NVR_ERR_INVALID_ARG, "retention: %d heads in groups of %d", a.H, a.qk_share);
    if (a.v_ones < 0 || a.v_ones >= a.Dv) return nvr::fail(NVR_ERR_INVALID_ARG, "retention: %d of %d value columns are ones", a.v_ones, a.Dv);
    if (!gated && !a.tok_gate && !a.decay) return nvr::fail(NVR_ERR_INVALID_ARG, "retention: no decay");
#define NVR_RET(R_)                                                                                  \
    do {                                                                                             \
        if (gated && a.bonus) { if (bf16) retention_seq_kernel<R_, bf16_t, 2><<<grid, dim3(256), 0, s>>>(a, b);   \
                                else retention_seq_kernel<R_, float, 2><<<grid, dim3(256), 0, s>>>(a, b); }       \
        else if (gated) { if (bf16) retention_seq_kernel<R_, bf16_t, 1><<<grid, dim3(256), 0, s>>>(a, b);   \
                     else retention_seq_kernel<R_, float, 1><<<grid, dim3(256), 0, s>>>(a, b); }       \
        else if (bf16) retention_seq_kernel<R_, bf16_t, 0><<<grid, dim3(256), 0, s>>>(a, b);     \
        else retention_seq_kernel<R_, float, 0><<<grid, dim3(256), 0, s>>>(a, b);                \
    } while (0)
    const size_t lds = ((size_t)(gated ? 3 : 2) * 16 * a.D + 16 * 32 + 16 * 8 * 32 + 32 + 128) * 4;
    if (a.D <= 256 && lds <= 64 * 1024) {                 // (beyond: the token-by-token form, whose LDS does not grow with the key size)
        const dim3 grid((unsigned)b.B, (unsigned)a.H, (unsigned)(((a.tok_gate && a.v_ones == 1 ? a.Dv - 1 : a.Dv) + 31) / 32));   // (a single column of ones rides in the first block)
#define NVR_RETB(R_)                                                                                 \
    do {                                                                                             \
        if (gated && a.bonus) { if (bf16) retention_block_kernel<R_, bf16_t, 2><<<grid, dim3(256), lds, s>>>(a, b);   \
                                else retention_block_kernel<R_, float, 2><<<grid, dim3(256), lds, s>>>(a, b); }       \
        else if (gated) { if (bf16) retention_block_kernel<R_, bf16_t, 1><<<grid, dim3(256), lds, s>>>(a, b);   \
                     else retention_block_kernel<R_, float, 1><<<grid, dim3(256), lds, s>>>(a, b); }       \
        else if (bf16) retention_block_kernel<R_, bf16_t, 0><<<grid, dim3(256), lds, s>>>(a, b); \
        else retention_block_kernel<R_, float, 0><<<grid, dim3(256), lds, s>>>(a, b);            \
    } while (0)
        if (rows <= 8) NVR_RETB(8);
        else if (rows <= 16) NVR_RETB(16);
        else NVR_RETB(32);
#undef NVR_RETB
        return launched("retention");
    }
    if (rows <= 8) NVR_RET(8);
    else if (rows <= 16) NVR_RET(16);
    else if (rows <= 32) NVR_RET(32);
    else NVR_RET(64);
#undef NVR_RET
    return launched("retention");
}

int head_norm_gate(const float *o, const void *gate, int64_t ldg, int64_t gcol, int64_t T, int64_t H, int64_t Dv, float eps, const float *w, void *out, int64_t ldo,
                   bool bf16, hipStream_t s, bool w_heads) {
    if (T == 0) return 0;
    const dim3 grid((unsigned)T);
    if (bf16) head_norm_gate_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(o, (const bf16_t *)gate, ldg, gcol, (int)H, (int)Dv, eps, w, (bf16_t *)out, ldo, w_heads ? 1 : 0);
    else head_norm_gate_kernel<float><<<grid, dim3(256), 0, s>>>(o, (const float *)gate, ldg, gcol, (int)H, (int)Dv, eps, w, (float *)out, ldo, w_heads ? 1 : 0);
    return launched("head_norm_gate");
}

int clamped_glu(const void *gu, int64_t T, int64_t F, float limit, float alpha, void *out, int64_t ldo, bool bf16, hipStream_t s) {
    if (T * F == 0) return 0;
    if (bf16 && F % 8 == 0 && ldo % 8 == 0 && ((uintptr_t)gu | (uintptr_t)out) % 16 == 0) {
        clamped_glu8_kernel<<<dim3((unsigned)((T * (F / 8) + 255) / 256)), dim3(256), 0, s>>>((const bf16_t *)gu, T, F, limit, alpha, (bf16_t *)out, ldo);
        return launched("clamped_glu");
    }
    const dim3 grid((unsigned)((T * F + 255) / 256));
    if (bf16) clamped_glu_kernel<bf16_t><<<grid, dim3(256), 0, s>>>((const bf16_t *)gu, T, F, limit, alpha, (bf16_t *)out, ldo);
    else clamped_glu_kernel<float><<<grid, dim3(256), 0, s>>>((const float *)gu, T, F, limit, alpha, (float *)out, ldo);
    return launched("clamped_glu");
}

int axpy(float *x, const void *y, bool bf16, float mult, int64_t n, hipStream_t s) {
    if (n == 0) return 0;
    if (bf16) axpy_kernel<bf16_t><<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s>>>(x, (const bf16_t *)y, mult, n);
    else axpy_kernel<float><<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s>>>(x, (const float *)y, mult, n);
    return launched("axpy");
}

int norm_rows(const float *x, const int32_t *rows, int64_t R, int64_t W, float eps, float g, void *out, bool bf16, hipStream_t s) {
    if (R == 0) return 0;
    if (bf16) norm_rows_kernel<bf16_t><<<dim3((unsigned)R), dim3(256), 0, s>>>(x, rows, (int)W, eps, g, (bf16_t *)out);
    else norm_rows_kernel<float><<<dim3((unsigned)R), dim3(256), 0, s>>>(x, rows, (int)W, eps, g, (float *)out);
    return launched("norm_rows");
}

int gemm_any(const void *a, int64_t lda, const void *w, int64_t T, int64_t K, int64_t N, void *y, bool y_f32, bool bf16, hipStream_t s) {
    if (T == 0 || N == 0) return 0;
    const dim3 grid((unsigned)((N + 15) / 16), (unsigned)((T + 15) / 16));
    if (bf16 && y_f32) gemm_any_kernel<bf16_t, float><<<grid, dim3(256), 0, s>>>((const bf16_t *)a, lda, (const bf16_t *)w, (int)T, (int)K, (int)N, (float *)y);
    else if (bf16) gemm_any_kernel<bf16_t, bf16_t><<<grid, dim3(256), 0, s>>>((const bf16_t *)a, lda, (const bf16_t *)w, (int)T, (int)K, (int)N, (bf16_t *)y);
    else gemm_any_kernel<float, float><<<grid, dim3(256), 0, s>>>((const float *)a, lda, (const float *)w, (int)T, (int)K, (int)N, (float *)y);
    return launched("gemm_any");
}

}}  // namespace nvr::kl
