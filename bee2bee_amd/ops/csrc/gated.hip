// Memory-bound kernels of the gated parallel-form layer stacks
//   x += sigmoid(g1) * mixer(h) + sigmoid(g2) * ffn(h),  h = unit(x) * w:
// the gated residual update fused with the next norm, the mean of two normed
// branch outputs, a weighted norm on a column slice, the exact gelu, rotation
// in either pair layout with the paged key/value store, and the minGRU
// recurrence (direct and segment-parallel).
//
// Every kernel is instantiated for bf16 (ushort bits) and fp32 activations;
// the residual stream, norm statistics, rotation angles, recurrence gates
// and state are fp32 in both.
#include "common.h"

#include <algorithm>

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

// VEC consecutive elements <-> floats; VEC = 4 moves 16 B (fp32) or 8 B
// (bf16) per lane.
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

DEV_INLINE float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }

constexpr int GA_THREADS = 256;

// sum over the workgroup; red: LDS [GA_THREADS / WAVE]; every thread gets it
DEV_INLINE float block_sum(float v, float* red) {
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    v = wave_sum(v);
    __syncthreads();            // earlier readers of red are done
    if (lane == 0) red[wid] = v;
    __syncthreads();
    float t = 0.f;
    for (int w = 0; w < (int)(blockDim.x / WAVE); ++w) t += red[w];
    return t;
}

// ------------------------------------------------ gated residual + norm
// resid += sigmoid(g1) * y1   (y1 given)
// resid += sigmoid(g2) * y2   (y2 given)
// resid += extra              (extra given)
// out    = unit(resid) * w    (out given)
// One workgroup per row; the updated row is held in LDS between the two
// passes, so every operand crosses HBM once. g1, g2 are column slices of a
// wider projection (row strides gs1, gs2).
template <typename YT, typename OT, int VEC>
__global__ void __launch_bounds__(GA_THREADS)
gated_add_rmsnorm_kernel(float* __restrict__ resid, const YT* __restrict__ y1,
                         const YT* __restrict__ g1, long gs1,
                         const YT* __restrict__ y2,
                         const YT* __restrict__ g2, long gs2,
                         const float* __restrict__ extra,
                         const float* __restrict__ w, OT* __restrict__ out,
                         int W, float eps) {
    extern __shared__ __attribute__((aligned(16))) float ga_row[];
    __shared__ float red[GA_THREADS / WAVE];
    const long t = blockIdx.x;
    float* rr = resid + t * (long)W;
    float ss = 0.f;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        float v[VEC];
        ldv<float, VEC>(rr + i, v);
        if (y1) {
            float a[VEC], g[VEC];
            ldv<YT, VEC>(y1 + t * (long)W + i, a);
            ldv<YT, VEC>(g1 + t * gs1 + i, g);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] += a[j] * sigmoid_f(g[j]);
        }
        if (y2) {
            float a[VEC], g[VEC];
            ldv<YT, VEC>(y2 + t * (long)W + i, a);
            ldv<YT, VEC>(g2 + t * gs2 + i, g);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] += a[j] * sigmoid_f(g[j]);
        }
        if (extra) {
            float e[VEC];
            ldv<float, VEC>(extra + t * (long)W + i, e);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] += e[j];
        }
        if (y1 || y2 || extra) stv<float, VEC>(rr + i, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            ga_row[i + j] = v[j];
            ss += v[j] * v[j];
        }
    }
    if (!out) return;
    const float r = 1.f / sqrtf(block_sum(ss, red) / (float)W + eps);
    OT* orow = out + t * (long)W;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        float v[VEC], wv[VEC];
        ldv<float, VEC>(w + i, wv);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = ga_row[i + j] * r * wv[j];
        stv<OT, VEC>(orow + i, v);
    }
}

// out = (unit(a) * wa + unit(b) * wb) / 2 over rows [T, W]; workgroup per
// row, both rows in LDS between the passes.
template <typename T, int VEC>
__global__ void __launch_bounds__(GA_THREADS)
pair_rmsnorm_mean_kernel(const T* __restrict__ a, const float* __restrict__ wa,
                         const T* __restrict__ b, const float* __restrict__ wb,
                         T* __restrict__ out, int W, float eps) {
    extern __shared__ __attribute__((aligned(16))) float pm_rows[];
    __shared__ float red[GA_THREADS / WAVE];
    float* ra = pm_rows;
    float* rb = pm_rows + W;
    const long t = blockIdx.x;
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        float x[VEC], y[VEC];
        ldv<T, VEC>(a + t * (long)W + i, x);
        ldv<T, VEC>(b + t * (long)W + i, y);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            ra[i + j] = x[j];
            rb[i + j] = y[j];
            sa += x[j] * x[j];
            sb += y[j] * y[j];
        }
    }
    const float qa = 0.5f / sqrtf(block_sum(sa, red) / (float)W + eps);
    const float qb = 0.5f / sqrtf(block_sum(sb, red) / (float)W + eps);
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        float u[VEC], v[VEC], o[VEC];
        ldv<float, VEC>(wa + i, u);
        ldv<float, VEC>(wb + i, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            o[j] = ra[i + j] * qa * u[j] + rb[i + j] * qb * v[j];
        stv<T, VEC>(out + t * (long)W + i, o);
    }
}

// unit(x) * w on a column slice (row stride xs) -> contiguous [T, N]; one
// wave per row, the second read hits L2.
template <typename T>
__global__ void __launch_bounds__(GA_THREADS)
slice_rmsnorm_kernel(const T* __restrict__ x, long xs,
                     const float* __restrict__ w, T* __restrict__ out, long Tn,
                     int N, float eps) {
    const long t = (long)blockIdx.x * (GA_THREADS / WAVE) + threadIdx.x / WAVE;
    if (t >= Tn) return;                  // no workgroup barrier below
    const int lane = threadIdx.x % WAVE;
    const T* xr = x + t * xs;
    float ss = 0.f;
    for (int i = lane; i < N; i += WAVE) {
        const float v = ldf(xr + i);
        ss += v * v;
    }
    const float r = 1.f / sqrtf(wave_sum(ss) / (float)N + eps);
    for (int i = lane; i < N; i += WAVE)
        stf(out + t * (long)N + i, ldf(xr + i) * r * w[i]);
}

// exact gelu, x/2 (1 + erf(x / sqrt 2)), element-wise on a contiguous buffer
template <typename T>
__global__ void gelu_erf_kernel(const T* __restrict__ x, T* __restrict__ y,
                                long n) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (long)gridDim.x * blockDim.x) {
        const float v = ldf(x + i);
        stf(y + i, 0.5f * v * (1.f + erff(v * 0.70710678118654752f)));
    }
}

// ----------------------------------------- rotation + key/value page store
// Workgroup per (token, four heads), a wave per head: H query heads, G key
// heads, G value heads. Query: rotate(q) * q_mult -> q_out (which may be q
// itself). Key: rotate(k) -> k_cache [n_blocks, G, bs, D]. Value: v ->
// v_cache [n_blocks, G, bs, Dv]. The rotation covers the first `dims`
// coordinates (cos/sin fp32 tables [max_pos, dims/2]); INTER pairs
// coordinate 2i with 2i+1, otherwise i with i + dims/2. Inputs are TIN
// (fp32 when they come out of a convolution), outputs T.
constexpr int RS_MAXD = 512;
template <typename TIN, typename T, bool INTER>
__global__ void __launch_bounds__(256)
rope_store_kernel(const TIN* q, long q_tok, T* q_out, long qo_tok, int H, const TIN* __restrict__ k, long k_tok,
                  const TIN* __restrict__ v, long v_tok, int G, int D, int Dv,
                  int dims, const int* __restrict__ positions,
                  const float* __restrict__ cos_t,
                  const float* __restrict__ sin_t, float q_mult,
                  T* __restrict__ k_cache, T* __restrict__ v_cache, int bs,
                  const int* __restrict__ slot_mapping) {
    __shared__ float buf[4][RS_MAXD];
    const long t = blockIdx.x;
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int pos = positions[t];
    const int half = dims / 2;
    const int slot = slot_mapping[t];
    const long blk = slot / bs, off = slot % bs;
    float* nb = buf[wid];
    // no workgroup barrier below, so waves past the end just leave
    const int hh = blockIdx.y * 4 + wid;
    if (hh >= H + 2 * G) return;
    if (hh >= H + G) {              // value head: copy into its page
        const int g = hh - H - G;
        const TIN* src = v + t * v_tok + (long)g * Dv;
        T* dst = v_cache + ((blk * G + g) * bs + off) * Dv;
        for (int i = lane; i < Dv; i += WAVE) stf(dst + i, ldf(src + i));
        return;
    }
    const bool is_q = hh < H;
    const int g = hh - H;
    const TIN* src = is_q ? q + t * q_tok + (long)hh * D
                          : k + t * k_tok + (long)g * D;
    for (int i = lane; i < D; i += WAVE) nb[i] = ldf(src + i);
    WAVE_LDS_SYNC();
    T* dst = is_q ? q_out + t * qo_tok + (long)hh * D
                  : k_cache + ((blk * G + g) * bs + off) * D;
    const float mult = is_q ? q_mult : 1.f;
    for (int i = lane; i < D; i += WAVE) {
        float y = nb[i];
        if (i < dims) {
            int j, ip;
            bool first;
            if (INTER) {
                j = i >> 1;
                ip = i ^ 1;
                first = (i & 1) == 0;
            } else {
                first = i < half;
                j = first ? i : i - half;
                ip = first ? i + half : i - half;
            }
            const float yp = nb[ip];
            const float cs = cos_t[(long)pos * half + j];
            const float sn = sin_t[(long)pos * half + j];
            y = first ? y * cs - yp * sn : y * cs + yp * sn;
        }
        stf(dst + i, y * mult);
    }
}

// ----------------------------------------------------------------- minGRU
// S_t = (1 - a_t) S_(t-1) + a_t c_t per channel, a = sigmoid(z), c = x + 1/2
// (x >= 0) or sigmoid(x); out_t = S_t * silu(g_t). z, x, g are column slices
// (row strides zs, xs, gs) of the input projection; state [n_slots, N] fp32.
constexpr int MG_SEG = 64;      // tokens per segment of the parallel form

DEV_INLINE void mg_step(float z, float x, float& S) {
    const float a = sigmoid_f(z);
    const float c = x >= 0.f ? x + 0.5f : sigmoid_f(x);
    S = (1.f - a) * S + a * c;
}
DEV_INLINE float silu_g(float g) { return g / (1.f + expf(-g)); }

// Direct form: thread = (chunk, channel), tokens in order from the carried
// state (zero, without reading the slot, when the chunk starts at position
// 0). Decode steps and short portions.
template <typename T>
__global__ void __launch_bounds__(256)
min_gru_kernel(const T* __restrict__ z, long zs, const T* __restrict__ x,
               long xs, const T* __restrict__ g, long gs,
               float* __restrict__ state, const int* __restrict__ state_slots,
               const int* __restrict__ cu, const int* __restrict__ positions,
               T* __restrict__ out, long os, int N) {
    const int b = blockIdx.x;
    const int n = blockIdx.y * blockDim.x + threadIdx.x;
    if (n >= N) return;
    const int lo = cu[b], hi = cu[b + 1];
    if (hi <= lo) return;
    float* st = state + (long)state_slots[b] * N + n;
    float S = positions[lo] == 0 ? 0.f : *st;
    for (int t = lo; t < hi; ++t) {
        mg_step(ldf(z + t * zs + n), ldf(x + t * xs + n), S);
        stf(out + t * os + n, S * silu_g(ldf(g + t * gs + n)));
    }
    *st = S;
}

// segment index -> (chunk, first row, end row); false when out of range
DEV_INLINE bool mg_segment(const int* __restrict__ cu, int B, int seg,
                           int* b_out, int* lo, int* hi) {
    int first = 0;
    for (int b = 0; b < B; ++b) {
        const int len = cu[b + 1] - cu[b];
        const int n = (len + MG_SEG - 1) / MG_SEG;
        if (seg < first + n) {
            *b_out = b;
            *lo = cu[b] + (seg - first) * MG_SEG;
            *hi = min(cu[b + 1], *lo + MG_SEG);
            return true;
        }
        first += n;
    }
    return false;
}

// Segment-parallel form for long portions. The recurrence is linear in S,
// so a segment's end state is P * S_start + L with P = prod (1 - a_t) and L
// the end state reached from zero:
//   phase 1: (P, L) of every segment, in parallel        -> ws_p, ws_l
//   phase 2: per (chunk, channel), walk the chunk's segments in order:
//            ws_l[seg] <- state at the segment's start; the slot gets the
//            chunk's end state
//   phase 3: every segment again from its true start state, writing out.
template <typename T, int PHASE>
__global__ void __launch_bounds__(256)
min_gru_seg_kernel(const T* __restrict__ z, long zs, const T* __restrict__ x,
                   long xs, const T* __restrict__ g, long gs,
                   const int* __restrict__ cu, int B,
                   float* __restrict__ ws_p, float* __restrict__ ws_l,
                   T* __restrict__ out, long os, int N) {
    const int n = blockIdx.y * blockDim.x + threadIdx.x;
    int b, lo, hi;
    if (!mg_segment(cu, B, blockIdx.x, &b, &lo, &hi) || n >= N) return;
    const long at = (long)blockIdx.x * N + n;
    if (PHASE == 1) {
        float P = 1.f, S = 0.f;
        for (int t = lo; t < hi; ++t) {
            const float zz = ldf(z + t * zs + n);
            P *= 1.f - sigmoid_f(zz);
            mg_step(zz, ldf(x + t * xs + n), S);
        }
        ws_p[at] = P;
        ws_l[at] = S;
    } else {
        float S = ws_l[at];
        for (int t = lo; t < hi; ++t) {
            mg_step(ldf(z + t * zs + n), ldf(x + t * xs + n), S);
            stf(out + t * os + n, S * silu_g(ldf(g + t * gs + n)));
        }
    }
}

__global__ void __launch_bounds__(256)
min_gru_scan_kernel(const int* __restrict__ cu,
                    const int* __restrict__ positions,
                    float* __restrict__ state,
                    const int* __restrict__ state_slots,
                    const float* __restrict__ ws_p, float* __restrict__ ws_l,
                    int N) {
    const int b = blockIdx.x;
    const int n = blockIdx.y * blockDim.x + threadIdx.x;
    if (n >= N) return;
    const int lo = cu[b], hi = cu[b + 1];
    if (hi <= lo) return;
    int first = 0;
    for (int i = 0; i < b; ++i)
        first += (cu[i + 1] - cu[i] + MG_SEG - 1) / MG_SEG;
    const int nseg = (hi - lo + MG_SEG - 1) / MG_SEG;
    float* st = state + (long)state_slots[b] * N + n;
    float S = positions[lo] == 0 ? 0.f : *st;
    for (int s = 0; s < nseg; ++s) {
        const long at = (long)(first + s) * N + n;
        const float P = ws_p[at], L = ws_l[at];
        ws_l[at] = S;
        S = P * S + L;
    }
    *st = S;
}

// ------------------------------------------------ group-limited routing
// One thread per token; its E scores (and group scores) live in LDS at
// stride blockDim, so neighbouring threads never share a bank. scores =
// sigmoid(logit) or softmax over all experts; a group's score is the sum of
// its group_top largest scores; experts outside the best `keep` groups
// cannot be chosen; the top_k best remaining scores are the weights, as they
// are, in descending order (ties: the lower index first).
constexpr int GT_THREADS = 64;
__global__ void __launch_bounds__(GT_THREADS)
group_topk_gate_kernel(const float* __restrict__ logits,
                       float* __restrict__ w_out, int* __restrict__ idx_out,
                       long T, int E, int top_k, int n_groups, int keep,
                       int group_top, int sigmoid) {
    extern __shared__ __attribute__((aligned(16))) float gt_s[];
    const long t = (long)blockIdx.x * GT_THREADS + threadIdx.x;
    if (t >= T) return;                    // no workgroup barrier below
    float* sc = gt_s + threadIdx.x;                       // [E]
    float* gsc = gt_s + (long)E * GT_THREADS + threadIdx.x;  // [n_groups]
    const int st = GT_THREADS;
    const float* z = logits + t * E;
    if (sigmoid) {
        for (int e = 0; e < E; ++e) sc[e * st] = sigmoid_f(z[e]);
    } else {
        float m = -INFINITY, sum = 0.f;
        for (int e = 0; e < E; ++e) m = fmaxf(m, z[e]);
        for (int e = 0; e < E; ++e) {
            const float x = expf(z[e] - m);
            sc[e * st] = x;
            sum += x;
        }
        for (int e = 0; e < E; ++e) sc[e * st] /= sum;
    }
    const int gs = E / n_groups;
    const bool limited = n_groups > 1 && keep < n_groups;
    if (limited) {
        const int gt = min(max(group_top, 1), gs);
        for (int g = 0; g < n_groups; ++g) {
            // sum of the gt largest: each pass takes the largest score that
            // is below the last one taken (or equal, at a higher index)
            float total = 0.f, last = INFINITY;
            int last_i = -1;
            for (int it = 0; it < gt; ++it) {
                float best = -1.f;
                int bi = -1;
                for (int j = 0; j < gs; ++j) {
                    const float x = sc[(g * gs + j) * st];
                    const bool open = x < last || (x == last && j > last_i);
                    if (open && x > best) { best = x; bi = j; }
                }
                total += best;
                last = best;
                last_i = bi;
            }
            gsc[g * st] = total;
        }
        for (int it = 0; it < keep; ++it) {
            float best = -1.f;
            int bg = 0;
            for (int g = 0; g < n_groups; ++g) {
                const float x = gsc[g * st];
                if (x > best) { best = x; bg = g; }
            }
            gsc[bg * st] = -2.f;           // kept
        }
    }
    for (int it = 0; it < top_k; ++it) {
        float best = -1.f;
        int be = 0;
        for (int e = 0; e < E; ++e) {
            if (limited && gsc[(e / gs) * st] != -2.f) continue;
            const float x = sc[e * st];
            if (x > best) { best = x; be = e; }
        }
        w_out[t * top_k + it] = best;
        idx_out[t * top_k + it] = be;
        sc[be * st] = -1.f;                // taken
    }
}

}  // namespace

// ---------------------------------------------------------------- launchers
// yc / oc / c: 0 = bf16, 1 = fp32. vec: rows, strides and base addresses
// allow 4-element accesses.

extern "C" void launch_gated_add_rmsnorm(
    float* resid, const void* y1, const void* g1, long gs1, const void* y2,
    const void* g2, long gs2, const float* extra, const float* w, void* out,
    long T, int W, float eps, int yc, int oc, int vec, hipStream_t s) {
    if (T == 0) return;
    const size_t smem = (size_t)W * sizeof(float);
#define GA_LAUNCH(YT, OT, V)                                                  \
    gated_add_rmsnorm_kernel<YT, OT, V><<<(unsigned)T, GA_THREADS, smem, s>>>(\
        resid, (const YT*)y1, (const YT*)g1, gs1, (const YT*)y2,              \
        (const YT*)g2, gs2, extra, w, (OT*)out, W, eps)
#define GA_PICK(YT, OT)                                                       \
    do {                                                                      \
        if (vec) GA_LAUNCH(YT, OT, 4);                                        \
        else GA_LAUNCH(YT, OT, 1);                                            \
    } while (0)
    if (yc && oc) GA_PICK(float, float);
    else if (yc) GA_PICK(float, unsigned short);
    else if (oc) GA_PICK(unsigned short, float);
    else GA_PICK(unsigned short, unsigned short);
#undef GA_PICK
#undef GA_LAUNCH
}

extern "C" void launch_pair_rmsnorm_mean(const void* a, const float* wa,
                                         const void* b, const float* wb,
                                         void* out, long T, int W, float eps,
                                         int c, int vec, hipStream_t s) {
    if (T == 0) return;
    const size_t smem = 2 * (size_t)W * sizeof(float);
#define PM_LAUNCH(TT, V)                                                      \
    pair_rmsnorm_mean_kernel<TT, V><<<(unsigned)T, GA_THREADS, smem, s>>>(    \
        (const TT*)a, wa, (const TT*)b, wb, (TT*)out, W, eps)
    if (c && vec) PM_LAUNCH(float, 4);
    else if (c) PM_LAUNCH(float, 1);
    else if (vec) PM_LAUNCH(unsigned short, 4);
    else PM_LAUNCH(unsigned short, 1);
#undef PM_LAUNCH
}

extern "C" void launch_slice_rmsnorm(const void* x, long xs, const float* w,
                                     void* out, long T, int N, float eps,
                                     int c, hipStream_t s) {
    if (T == 0) return;
    const int per = GA_THREADS / WAVE;
    const unsigned grid = (unsigned)((T + per - 1) / per);
    if (c)
        slice_rmsnorm_kernel<float><<<grid, GA_THREADS, 0, s>>>(
            (const float*)x, xs, w, (float*)out, T, N, eps);
    else
        slice_rmsnorm_kernel<unsigned short><<<grid, GA_THREADS, 0, s>>>(
            (const unsigned short*)x, xs, w, (unsigned short*)out, T, N, eps);
}

extern "C" void launch_gelu_erf(const void* x, void* y, long n, int c,
                                hipStream_t s) {
    if (n == 0) return;
    const unsigned grid = (unsigned)std::min<long>((n + 255) / 256, 8192);
    if (c)
        gelu_erf_kernel<float><<<grid, 256, 0, s>>>((const float*)x,
                                                    (float*)y, n);
    else
        gelu_erf_kernel<unsigned short><<<grid, 256, 0, s>>>(
            (const unsigned short*)x, (unsigned short*)y, n);
}

// in_f32: q/k/v inputs are fp32 (conv output) while q_out and the pages are
// the activation type c. Returns nonzero when a head size exceeds 512.
extern "C" int launch_rope_store(
    const void* q, long q_tok, void* q_out, long qo_tok, int H, const void* k,
    long k_tok, const void* v, long v_tok, int G, int D, int Dv, int dims,
    int inter, const int* positions, const float* cos_t, const float* sin_t,
    float q_mult, void* k_cache, void* v_cache, int bs,
    const int* slot_mapping, long T, int in_f32, int c, hipStream_t s) {
    if (D > RS_MAXD) return 1;
    if (T == 0) return 0;
    const dim3 grid((unsigned)T, (H + 2 * G + 3) / 4);
#define RS_LAUNCH(TIN, TT, I)                                                 \
    rope_store_kernel<TIN, TT, I><<<grid, 256, 0, s>>>(                       \
        (const TIN*)q, q_tok, (TT*)q_out, qo_tok, H, (const TIN*)k, k_tok,    \
        (const TIN*)v, v_tok, G, D, Dv, dims, positions, cos_t, sin_t,        \
        q_mult, (TT*)k_cache, (TT*)v_cache, bs, slot_mapping)
#define RS_PICK(TIN, TT)                                                      \
    do {                                                                      \
        if (inter) RS_LAUNCH(TIN, TT, true);                                  \
        else RS_LAUNCH(TIN, TT, false);                                       \
    } while (0)
    if (c) RS_PICK(float, float);
    else if (in_f32) RS_PICK(float, unsigned short);
    else RS_PICK(unsigned short, unsigned short);
#undef RS_PICK
#undef RS_LAUNCH
    return 0;
}

extern "C" int min_gru_segment_tokens() { return MG_SEG; }

// n_seg = 0: the direct form. n_seg > 0: an upper bound of the number of
// MG_SEG-token segments in the batch; ws_p and ws_l hold n_seg * N floats.
extern "C" void launch_min_gru(const void* z, long zs, const void* x, long xs,
                               const void* g, long gs, float* state,
                               const int* state_slots, const int* cu,
                               const int* positions, void* out, long os,
                               float* ws_p, float* ws_l, int n_seg, int B,
                               int N, int c, hipStream_t s) {
    if (B == 0 || N == 0) return;
    const unsigned cb = (N + 255) / 256;
    if (n_seg == 0) {
        const dim3 grid(B, cb);
        if (c)
            min_gru_kernel<float><<<grid, 256, 0, s>>>(
                (const float*)z, zs, (const float*)x, xs, (const float*)g, gs,
                state, state_slots, cu, positions, (float*)out, os, N);
        else
            min_gru_kernel<unsigned short><<<grid, 256, 0, s>>>(
                (const unsigned short*)z, zs, (const unsigned short*)x, xs,
                (const unsigned short*)g, gs, state, state_slots, cu,
                positions, (unsigned short*)out, os, N);
        return;
    }
    const dim3 sgrid(n_seg, cb), bgrid(B, cb);
#define MG_SEG_LAUNCH(TT, PH)                                                 \
    min_gru_seg_kernel<TT, PH><<<sgrid, 256, 0, s>>>(                         \
        (const TT*)z, zs, (const TT*)x, xs, (const TT*)g, gs, cu, B, ws_p,    \
        ws_l, (TT*)out, os, N)
    if (c) MG_SEG_LAUNCH(float, 1);
    else MG_SEG_LAUNCH(unsigned short, 1);
    min_gru_scan_kernel<<<bgrid, 256, 0, s>>>(cu, positions, state,
                                              state_slots, ws_p, ws_l, N);
    if (c) MG_SEG_LAUNCH(float, 3);
    else MG_SEG_LAUNCH(unsigned short, 3);
#undef MG_SEG_LAUNCH
}

// Returns nonzero when the scores of a workgroup's tokens do not fit LDS.
extern "C" int launch_group_topk_gate(const float* logits, float* w_out,
                                      int* idx_out, long T, int E, int top_k,
                                      int n_groups, int keep, int group_top,
                                      int sigmoid, hipStream_t s) {
    const size_t smem = (size_t)(E + n_groups) * GT_THREADS * sizeof(float);
    if (smem > 64 * 1024) return 1;
    if (T == 0) return 0;
    const unsigned grid = (unsigned)((T + GT_THREADS - 1) / GT_THREADS);
    group_topk_gate_kernel<<<grid, GT_THREADS, smem, s>>>(
        logits, w_out, idx_out, T, E, top_k, n_groups, keep, group_top,
        sigmoid);
    return 0;
}
