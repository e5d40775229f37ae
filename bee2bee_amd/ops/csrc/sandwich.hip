// Memory-bound kernels of the weighted-sandwich layer stacks
// (x += w_b * gnorm(f(w_a * gnorm(x))) with RMS norms taken over equal
// consecutive parts of a row): the grouped norm fused with the fp32 residual
// update and an optional per-pass step vector, "rotate, then unit-norm"
// query/key preparation with the paged key/value store, the PolyNorm
// activation and the plain silu gated-linear-unit.
//
// Every kernel is instantiated for bf16 (ushort bits) and fp32 activations;
// the residual stream, norm statistics and rotation angles are fp32 in both.
#include "common.h"

namespace {

template <typename T> DEV_INLINE float ldf(const T* p);
template <> DEV_INLINE float ldf<float>(const float* p) { return *p; }
template <> DEV_INLINE float ldf<unsigned short>(const unsigned short* p) {
    return bf2f(*p);
}
template <typename T> DEV_INLINE void stf(T* p, float v);
template <> DEV_INLINE void stf<float>(float* p, float v) { *p = v; }
template <> DEV_INLINE void stf<unsigned short>(unsigned short* p, float v) {
    *p = f2bf(v);
}

// VEC consecutive elements <-> floats. VEC = 4 moves 16 B (fp32) or 8 B
// (bf16) per lane and needs rows whose length is a multiple of 4.
template <typename T, int VEC> DEV_INLINE void ldv(const T* p, float* o);
template <> DEV_INLINE void ldv<float, 1>(const float* p, float* o) { o[0] = *p; }
template <> DEV_INLINE void ldv<unsigned short, 1>(const unsigned short* p, float* o) {
    o[0] = bf2f(*p);
}
template <> DEV_INLINE void ldv<float, 4>(const float* p, float* o) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(p);
    o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
}
template <> DEV_INLINE void ldv<unsigned short, 4>(const unsigned short* p, float* o) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    o[0] = bf2f((unsigned short)(w.x & 0xffffu));
    o[1] = bf2f((unsigned short)(w.x >> 16));
    o[2] = bf2f((unsigned short)(w.y & 0xffffu));
    o[3] = bf2f((unsigned short)(w.y >> 16));
}
template <typename T, int VEC> DEV_INLINE void stv(T* p, const float* o);
template <> DEV_INLINE void stv<float, 1>(float* p, const float* o) { *p = o[0]; }
template <> DEV_INLINE void stv<unsigned short, 1>(unsigned short* p, const float* o) {
    *p = f2bf(o[0]);
}
template <> DEV_INLINE void stv<float, 4>(float* p, const float* o) {
    *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
}
template <> DEV_INLINE void stv<unsigned short, 4>(unsigned short* p, const float* o) {
    uint2 w;
    w.x = (unsigned int)f2bf(o[0]) | ((unsigned int)f2bf(o[1]) << 16);
    w.y = (unsigned int)f2bf(o[2]) | ((unsigned int)f2bf(o[3]) << 16);
    *reinterpret_cast<uint2*>(p) = w;
}

constexpr int GN_MAXG = 64;     // parts of a row
constexpr int GN_MAXW = 16;     // waves per workgroup

// Sum of squares of each of `groups` equal parts of buf[0..W) (LDS, written
// and synchronized by the caller) -> sums[g] in LDS, visible to every
// thread on return. red: LDS [GN_MAXW * GN_MAXG].
DEV_INLINE void group_sumsq(const float* buf, int W, int groups, float* red,
                            float* sums) {
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int nw = (blockDim.x + WAVE - 1) / WAVE;
    const int gw = W / groups;
    for (int g = 0; g < groups; ++g) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < gw; i += blockDim.x) {
            const float v = buf[g * gw + i];
            ss += v * v;
        }
        ss = wave_sum(ss);
        if (lane == 0) red[wid * GN_MAXG + g] = ss;
    }
    __syncthreads();
    if (threadIdx.x < groups) {
        float total = 0.f;
        for (int w = 0; w < nw; ++w) total += red[w * GN_MAXG + threadIdx.x];
        sums[threadIdx.x] = total;
    }
    __syncthreads();
}

// ------------------------------------------------ grouped weighted norm
// resid += gnorm(y) * w_post   (y given)
// resid += step                (step given)
// out    = gnorm(resid) * w_pre (out given)
// gnorm: each of `groups` equal consecutive parts of the row divided by its
// own sqrt(mean^2 + eps). One workgroup per row; the row (and y) are held
// in LDS between the passes, so every operand crosses HBM once.
// VEC = 4 needs the part width (W / groups) to be a multiple of 4.
template <typename YT, typename OT, int VEC>
__global__ void add_group_rmsnorm_kernel(float* __restrict__ resid,
                                         const YT* __restrict__ y,
                                         const float* __restrict__ w_post,
                                         const float* __restrict__ step,
                                         const float* __restrict__ w_pre,
                                         OT* __restrict__ out, int W,
                                         int groups, float eps) {
    extern __shared__ __attribute__((aligned(16))) char smem_raw[];
    float* row = reinterpret_cast<float*>(smem_raw);     // [W]
    float* yrow = row + W;                               // [W] when y
    __shared__ float red[GN_MAXW * GN_MAXG];
    __shared__ float sums[GN_MAXG];
    const long t = blockIdx.x;
    const int gw = W / groups;
    float* rr = resid + t * (long)W;
    if (y) {
        const YT* yr = y + t * (long)W;
        for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
            float v[VEC];
            ldv<YT, VEC>(yr + i, v);
#pragma unroll
            for (int j = 0; j < VEC; ++j) yrow[i + j] = v[j];
        }
        __syncthreads();
        group_sumsq(yrow, W, groups, red, sums);
    }
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        float v[VEC];
        ldv<float, VEC>(rr + i, v);
        if (y) {
            const float r = 1.f / sqrtf(sums[i / gw] / (float)gw + eps);
            float wv[VEC];
            ldv<float, VEC>(w_post + i, wv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] += yrow[i + j] * r * wv[j];
        }
        if (step) {
            float sv[VEC];
            ldv<float, VEC>(step + i, sv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] += sv[j];
        }
        if (y || step) stv<float, VEC>(rr + i, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) row[i + j] = v[j];
    }
    if (!out) return;
    __syncthreads();
    group_sumsq(row, W, groups, red, sums);
    OT* orow = out + t * (long)W;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        const float r = 1.f / sqrtf(sums[i / gw] / (float)gw + eps);
        float v[VEC], wv[VEC];
        ldv<float, VEC>(w_pre + i, wv);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = row[i + j] * r * wv[j];
        stv<OT, VEC>(orow + i, v);
    }
}

// --------------------------------- rotation, unit norm, key/value page store
// Workgroup per (token, four heads), a wave per head: H query heads, G key
// heads, G value heads. Query: q <- unit(rotate(q)) * q_mult in place. Key:
// unit(rotate(k)) -> k_cache [n_blocks, G, bs, D]. Value: v -> v_cache
// [n_blocks, G, bs, Dv]. The rotation pairs coordinate i with i + dims/2
// over the first `dims` coordinates (cos/sin fp32 tables [max_pos, dims/2],
// any magnitude factor already inside); unit = x / sqrt(mean(x^2) + eps),
// taken AFTER the rotation, no weight.
constexpr int RU_MAXD = 512;
template <typename T>
__global__ void __launch_bounds__(256)
rope_unit_store_kernel(T* __restrict__ q, long q_tok, int H,
                       const T* __restrict__ k, long k_tok,
                       const T* __restrict__ v, long v_tok, int G, int D,
                       int Dv, float eps, int dims,
                       const int* __restrict__ positions,
                       const float* __restrict__ cos_t,
                       const float* __restrict__ sin_t, float q_mult,
                       T* __restrict__ k_cache, T* __restrict__ v_cache,
                       int bs, const int* __restrict__ slot_mapping) {
    __shared__ float buf[4][RU_MAXD];
    const long t = blockIdx.x;
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int pos = positions[t];
    const int half = dims / 2;
    const int slot = slot_mapping[t];
    const long blk = slot / bs, off = slot % bs;
    float* nb = buf[wid];
    // one head per wave: blockIdx.y walks the H + 2G heads four at a time
    // (no workgroup barrier below, so waves past the end just leave)
    const int hh = blockIdx.y * 4 + wid;
    if (hh >= H + 2 * G) return;
    if (hh >= H + G) {              // value head: plain copy into its page
        const int g = hh - H - G;
        const T* src = v + t * v_tok + (long)g * Dv;
        T* dst = v_cache + ((blk * G + g) * bs + off) * Dv;
        for (int i = lane; i < Dv; i += WAVE) dst[i] = src[i];
        return;
    }
    const bool is_q = hh < H;
    const int g = hh - H;
    const T* src = is_q ? q + t * q_tok + (long)hh * D
                        : k + t * k_tok + (long)g * D;
    for (int i = lane; i < D; i += WAVE) nb[i] = ldf(src + i);
    WAVE_LDS_SYNC();
    // rotated coordinates of this lane (D <= RU_MAXD: at most 8 each)
    float yv[RU_MAXD / WAVE];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < RU_MAXD / WAVE; ++c) {
        const int i = lane + c * WAVE;
        float y = 0.f;
        if (i < D) {
            y = nb[i];
            if (i < dims) {
                const int j = i < half ? i : i - half;
                const float yp = nb[i < half ? i + half : i - half];
                const float cs = cos_t[(long)pos * half + j];
                const float sn = sin_t[(long)pos * half + j];
                y = i < half ? y * cs - yp * sn : y * cs + yp * sn;
            }
        }
        yv[c] = y;
        ss += y * y;
    }
    const float r = 1.f / sqrtf(wave_sum(ss) / (float)D + eps) *
                    (is_q ? q_mult : 1.f);
    T* dst = is_q ? q + t * q_tok + (long)hh * D
                  : k_cache + ((blk * G + g) * bs + off) * D;
#pragma unroll
    for (int c = 0; c < RU_MAXD / WAVE; ++c) {
        const int i = lane + c * WAVE;
        if (i < D) stf(dst + i, yv[c] * r);
    }
}

// -------------------------------------------------------------- PolyNorm
// Row-wise: out = a unit(z) + b unit(z^2) + c unit(z^3) + e with
// unit(x) = x / sqrt(mean(x^2) + eps) over the row and (a, b, c, e) = coef.
// Workgroup per row; the row is read twice (the second read hits L2).
template <typename T>
__global__ void polynorm_kernel(const T* __restrict__ z,
                                const float* __restrict__ coef,
                                T* __restrict__ out, int N, float eps) {
    __shared__ float red[3][GN_MAXW];
    const long t = blockIdx.x;
    const T* zr = z + t * (long)N;
    float s2 = 0.f, s4 = 0.f, s6 = 0.f;
    for (int i = threadIdx.x; i < N; i += blockDim.x) {
        const float x = ldf(zr + i);
        const float x2 = x * x;
        s2 += x2;
        s4 += x2 * x2;
        s6 += x2 * x2 * x2;
    }
    s2 = wave_sum(s2);
    s4 = wave_sum(s4);
    s6 = wave_sum(s6);
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    if (lane == 0) {
        red[0][wid] = s2;
        red[1][wid] = s4;
        red[2][wid] = s6;
    }
    __syncthreads();
    const int nw = (blockDim.x + WAVE - 1) / WAVE;
    float t2 = 0.f, t4 = 0.f, t6 = 0.f;
    for (int w = 0; w < nw; ++w) {
        t2 += red[0][w];
        t4 += red[1][w];
        t6 += red[2][w];
    }
    const float a = coef[0] / sqrtf(t2 / (float)N + eps);
    const float b = coef[1] / sqrtf(t4 / (float)N + eps);
    const float c = coef[2] / sqrtf(t6 / (float)N + eps);
    const float e = coef[3];
    T* orow = out + t * (long)N;
    for (int i = threadIdx.x; i < N; i += blockDim.x) {
        const float x = ldf(zr + i);
        const float x2 = x * x;
        stf(orow + i, a * x + b * x2 + c * x2 * x + e);
    }
}

// --------------------------------------------------------------- silu GLU
// [rows, 2I] -> [rows, I]: silu(gate) * up
template <typename T>
__global__ void silu_glu_kernel(const T* __restrict__ gu, T* __restrict__ y,
                                long rows, long I) {
    const long n = rows * I;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < n;
         idx += (long)gridDim.x * blockDim.x) {
        const long r = idx / I, c = idx - r * I;
        const float g = ldf(gu + r * 2 * I + c);
        const float u = ldf(gu + r * 2 * I + I + c);
        stf(y + idx, g / (1.f + expf(-g)) * u);
    }
}

static inline int row_threads(int W) {
    int th = 64;
    while (th < W && th < 1024) th <<= 1;
    return th > 256 && W < 4096 ? 256 : th;
}

}  // namespace

// dtype codes: 0 = bf16 (ushort bits), 1 = fp32
// returns nonzero when groups does not divide W or exceeds 64
extern "C" int launch_add_group_rmsnorm(float* resid, const void* y,
                                        const float* w_post, const float* step,
                                        const float* w_pre, void* out, long T,
                                        int W, int groups, float eps,
                                        int y_f32, int out_f32,
                                        hipStream_t s) {
    if (groups < 1 || groups > GN_MAXG || W % groups) return 1;
    if (T == 0) return 0;
    const size_t sh = (size_t)W * sizeof(float) * (y ? 2 : 1);
    const bool vec = (W / groups) % 4 == 0;
    const int th = row_threads(vec ? W / 4 : W);
#define AGN(YT, OT)                                                           \
    do {                                                                      \
        if (vec)                                                              \
            add_group_rmsnorm_kernel<YT, OT, 4><<<T, th, sh, s>>>(            \
                resid, (const YT*)y, w_post, step, w_pre, (OT*)out, W,        \
                groups, eps);                                                 \
        else                                                                  \
            add_group_rmsnorm_kernel<YT, OT, 1><<<T, th, sh, s>>>(            \
                resid, (const YT*)y, w_post, step, w_pre, (OT*)out, W,        \
                groups, eps);                                                 \
    } while (0)
    if (y_f32 && out_f32) AGN(float, float);
    else if (y_f32) AGN(float, unsigned short);
    else if (out_f32) AGN(unsigned short, float);
    else AGN(unsigned short, unsigned short);
#undef AGN
    return 0;
}

// returns nonzero when a head size exceeds 512
extern "C" int launch_rope_unit_store(
    void* q, long q_tok, int H, const void* k, long k_tok, const void* v,
    long v_tok, int G, int D, int Dv, float eps, int dims,
    const int* positions, const float* cos_t, const float* sin_t,
    float q_mult, void* k_cache, void* v_cache, int bs,
    const int* slot_mapping, long T, int f32, hipStream_t s) {
    if (D > RU_MAXD) return 1;
    if (T == 0) return 0;
    const dim3 grid(T, (H + 2 * G + 3) / 4);
    if (f32)
        rope_unit_store_kernel<float><<<grid, 256, 0, s>>>(
            (float*)q, q_tok, H, (const float*)k, k_tok, (const float*)v,
            v_tok, G, D, Dv, eps, dims, positions, cos_t, sin_t, q_mult,
            (float*)k_cache, (float*)v_cache, bs, slot_mapping);
    else
        rope_unit_store_kernel<unsigned short><<<grid, 256, 0, s>>>(
            (unsigned short*)q, q_tok, H, (const unsigned short*)k, k_tok,
            (const unsigned short*)v, v_tok, G, D, Dv, eps, dims, positions,
            cos_t, sin_t, q_mult, (unsigned short*)k_cache,
            (unsigned short*)v_cache, bs, slot_mapping);
    return 0;
}

extern "C" void launch_polynorm(const void* z, const float* coef, void* out,
                                long T, int N, float eps, int f32,
                                hipStream_t s) {
    if (T == 0) return;
    const int th = row_threads(N);
    if (f32)
        polynorm_kernel<float><<<T, th, 0, s>>>((const float*)z, coef,
                                                (float*)out, N, eps);
    else
        polynorm_kernel<unsigned short><<<T, th, 0, s>>>(
            (const unsigned short*)z, coef, (unsigned short*)out, N, eps);
}

extern "C" void launch_silu_glu(const void* gu, void* y, long rows, long I,
                                int f32, hipStream_t s) {
    const long n = rows * I;
    if (n == 0) return;
    const int th = 256;
    long blocks = (n + th - 1) / th;
    if (blocks > 65536) blocks = 65536;
    if (f32)
        silu_glu_kernel<float><<<(int)blocks, th, 0, s>>>(
            (const float*)gu, (float*)y, rows, I);
    else
        silu_glu_kernel<unsigned short><<<(int)blocks, th, 0, s>>>(
            (const unsigned short*)gu, (unsigned short*)y, rows, I);
}
