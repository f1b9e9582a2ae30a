// layered.hip — kernels of layer-list models (kernels/layered.h): f32 residual stream, scalar-gain RMS norm + causal convolution in front
// of each sublayer, attention with distance penalty and sink, retention with f32 state, clamped gated feed-forward.  wave64, gfx950.
#include <hip/hip_runtime.h>
#include <math.h>
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

// ------------------------------------------------------------------------------------------------ K / V rows into the paged caches
template <class CT>
__global__ __launch_bounds__(256) void kv_store_kernel(const CT *__restrict__ proj, int64_t ld, int64_t kcol, int64_t vcol, Batch b, int G, int D, int Dv,
                                                       CT *__restrict__ kc, CT *__restrict__ vc) {
    const int t = blockIdx.x, sq = b.row_seq[t];
    const int p = b.start[sq] + (t - b.cu[sq]);
    const int blk = b.block_tables[(int64_t)sq * b.max_blocks + p / b.block_size];
    const int64_t row = (int64_t)blk * b.block_size + p % b.block_size;
    const CT *pr = proj + (int64_t)t * ld;
    for (int c = threadIdx.x; c < G * D; c += 256) kc[row * G * D + c] = pr[kcol + c];
    for (int c = threadIdx.x; c < G * Dv; c += 256) vc[row * G * Dv + c] = pr[vcol + c];
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
    const float r1 = a.r1 ? a.r1[h] : 0.f, r2 = a.r2 ? a.r2[h] : 0.f;
    float mx = a.sink ? a.sink[h] : -INFINITY;
    for (int j = threadIdx.x; j < ctx; j += 256) {
        const int64_t row = (int64_t)bt[j / b.block_size] * b.block_size + j % b.block_size;
        const int64_t base = (row * a.G + kvh) * a.D;
        float dot = 0.f;
        for (int d = 0; d < a.D; ++d) dot += qs[d] * ld_f(kc, base + d);
        float s = dot * a.scale;
        if (a.r1) s -= r1 * log1pf(r2 * (float)(i - j));
        sc[j] = s;
        mx = fmaxf(mx, s);
    }
    mx = block_max<256>(mx, red);
    float sum = 0.f;
    for (int j = threadIdx.x; j < ctx; j += 256) { const float e = expf(sc[j] - mx); sc[j] = e; sum += e; }
    sum = block_sum<256>(sum, red);                     // (its barriers also publish the weights)
    if (a.sink) sum += expf(a.sink[h] - mx);
    const float inv = 1.0f / sum;
    // values: column c by lanes, keys split over the 256 / CW groups
    float *part = sc + ctx;
    for (int cb = 0; cb < a.Dv; cb += 64) {
        const int c = cb + (threadIdx.x & 63), grp = threadIdx.x >> 6;
        float acc = 0.f;
        if (c < a.Dv)
            for (int j = grp; j < ctx; j += 4) {
                const int64_t row = (int64_t)bt[j / b.block_size] * b.block_size + j % b.block_size;
                acc += sc[j] * ld_f(vc, (row * a.G + kvh) * a.Dv + c);
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

// ------------------------------------------------------------------------------------------------ retention, token by token
// One workgroup per (sequence, head, block of 32 value columns): thread (c, part) keeps rows part, part + 8, ... of column c of the state in registers.
template <int RMAX, class PT>
__global__ __launch_bounds__(256) void retention_seq_kernel(RetentionArgs a, Batch b) {
    __shared__ float qs[2][512], ks[2][512], red[8][32];
    const int sq = blockIdx.x, h = blockIdx.y, cb = blockIdx.z * 32;
    const int c = cb + (threadIdx.x & 31), part = threadIdx.x >> 5;
    const int r0 = b.cu[sq], n = b.cu[sq + 1] - r0, st = b.start[sq];
    const int D = a.D, Dv = a.Dv, half = a.rot_dims / 2;
    const float dec = a.decay[h];
    float *S = a.state + (((int64_t)b.slot[sq] * a.H + h) * D) * Dv;
    const bool live = c < Dv;
    float s[RMAX];
#pragma unroll
    for (int r = 0; r < RMAX; ++r) { const int d = part + r * 8; s[r] = (st > 0 && live && d < D) ? S[(int64_t)d * Dv + c] : 0.f; }
    for (int i = 0; i < n; ++i) {
        const int t = r0 + i, buf = i & 1;
        const PT *pr = (const PT *)a.proj + (int64_t)t * a.ld;
        const PT *q = pr + a.qcol + (int64_t)h * D, *k = pr + a.kcol + (int64_t)h * D;
        for (int d = threadIdx.x; d < D; d += 256) {
            float qv = ld_f(q, d), kv = ld_f(k, d);
            if (d < a.rot_dims) {
                const int fi = d < half ? d : d - half;
                const float ang = (float)(st + i) * a.freq[fi];
                float sn, cs; sincosf(ang, &sn, &cs);
                if (d < half) { qv = qv * cs - ld_f(q, d + half) * sn; kv = kv * cs - ld_f(k, d + half) * sn; }
                else { qv = qv * cs + ld_f(q, d - half) * sn; kv = kv * cs + ld_f(k, d - half) * sn; }
            }
            qs[buf][d] = qv; ks[buf][d] = kv * a.kscale;
        }
        __syncthreads();
        const float v = live ? ld_f(pr, a.vcol + (int64_t)h * Dv + c) : 0.f;
        float o = 0.f;
#pragma unroll
        for (int r = 0; r < RMAX; ++r) {
            const int d = part + r * 8;
            if (d < D) { s[r] = dec * s[r] + ks[buf][d] * v; o += s[r] * qs[buf][d]; }
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

template <class OT>
__global__ __launch_bounds__(64) void head_norm_gate_kernel(const float *__restrict__ o, const OT *__restrict__ gate, int64_t ldg, int64_t gcol, int H, int Dv,
                                                            float eps, OT *__restrict__ out, int64_t ldo) {
    const int64_t t = blockIdx.x; const int h = blockIdx.y;
    const float *orow = o + (t * H + h) * Dv;
    float ss = 0.f;
    for (int c = threadIdx.x; c < Dv; c += 64) { const float v = orow[c]; ss += v * v; }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)Dv + eps);
    for (int c = threadIdx.x; c < Dv; c += 64) {
        const float g = ld_f(gate, t * ldg + gcol + (int64_t)h * Dv + c);
        st_f(out, t * ldo + (int64_t)h * Dv + c, orow[c] * r * (g / (1.0f + expf(-g))));
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
    const size_t lds = (size_t)taps * (size_t)W * 4;
    if (lds > kMaxLds) return nvr::fail(NVR_ERR_UNSUPPORTED, "norm_canon: %d taps of %ld channels do not fit LDS", taps, (long)W);
    if (bf16) norm_canon_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(256), lds, s>>>(x, b, (int)W, eps, taps, g1, w1, (bf16_t *)out1, g2, w2, (bf16_t *)out2, hist, slots);
    else norm_canon_kernel<float><<<dim3((unsigned)b.T), dim3(256), lds, s>>>(x, b, (int)W, eps, taps, g1, w1, (float *)out1, g2, w2, (float *)out2, hist, slots);
    return launched("norm_canon");
}

int kv_store(const void *proj, int64_t ld, int64_t kcol, int64_t vcol, const Batch &b, int64_t G, int64_t D, int64_t Dv, void *kc, void *vc, bool bf16,
             hipStream_t s) {
    if (b.T == 0) return 0;
    if (bf16) kv_store_kernel<bf16_t><<<dim3((unsigned)b.T), dim3(256), 0, s>>>((const bf16_t *)proj, ld, kcol, vcol, b, (int)G, (int)D, (int)Dv, (bf16_t *)kc, (bf16_t *)vc);
    else kv_store_kernel<float><<<dim3((unsigned)b.T), dim3(256), 0, s>>>((const float *)proj, ld, kcol, vcol, b, (int)G, (int)D, (int)Dv, (float *)kc, (float *)vc);
    return launched("kv_store");
}

int sink_attention(const SinkAttnArgs &a, const Batch &b, bool bf16, hipStream_t s) {
    if (b.T == 0) return 0;
    if (a.G < 1 || a.H % a.G) return nvr::fail(NVR_ERR_INVALID_ARG, "sink_attention: %d heads over %d key/value heads", a.H, a.G);
    const size_t lds = ((size_t)a.D + (size_t)b.max_ctx + 256) * 4;
    if (lds > kMaxLds) return nvr::fail(NVR_ERR_UNSUPPORTED, "sink_attention: a context of %d keys does not fit the score buffer", b.max_ctx);
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
#define NVR_RET(R_)                                                                                  \
    do {                                                                                             \
        if (bf16) retention_seq_kernel<R_, bf16_t><<<grid, dim3(256), 0, s>>>(a, b);                 \
        else retention_seq_kernel<R_, float><<<grid, dim3(256), 0, s>>>(a, b);                       \
    } while (0)
    if (rows <= 8) NVR_RET(8);
    else if (rows <= 16) NVR_RET(16);
    else if (rows <= 32) NVR_RET(32);
    else NVR_RET(64);
#undef NVR_RET
    return launched("retention");
}

int head_norm_gate(const float *o, const void *gate, int64_t ldg, int64_t gcol, int64_t T, int64_t H, int64_t Dv, float eps, void *out, int64_t ldo, bool bf16,
                   hipStream_t s) {
    if (T == 0) return 0;
    const dim3 grid((unsigned)T, (unsigned)H);
    if (bf16) head_norm_gate_kernel<bf16_t><<<grid, dim3(64), 0, s>>>(o, (const bf16_t *)gate, ldg, gcol, (int)H, (int)Dv, eps, (bf16_t *)out, ldo);
    else head_norm_gate_kernel<float><<<grid, dim3(64), 0, s>>>(o, (const float *)gate, ldg, gcol, (int)H, (int)Dv, eps, (float *)out, ldo);
    return launched("head_norm_gate");
}

int clamped_glu(const void *gu, int64_t T, int64_t F, float limit, float alpha, void *out, int64_t ldo, bool bf16, hipStream_t s) {
    if (T * F == 0) return 0;
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
