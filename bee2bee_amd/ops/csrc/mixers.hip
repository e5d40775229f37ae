// Sequence mixers of the hybrid layer stacks.
//
// latent_attn: windowed softmax attention over a paged cache that holds ONE
// row per token (normed latent | rotated key part) shared by all heads —
// the "absorbed" form: queries arrive already multiplied by the key
// up-projection, the output is the probability-weighted sum of latent rows
// (the value up-projection is applied afterwards as a batched GEMM).
// One wave per (token, head): lanes span the row's coordinates, keys are
// walked four at a time with an online softmax; scores, weights and
// accumulators are fp32. The same kernel serves prompt portions and decode
// rows: every row carries its own position and sequence. When a step has
// few rows (decode), the visible keys of each row are split over grid.z so
// the chip is filled, and a second kernel merges the (max, sum, partial)
// triples.
//
// lightning_attn: decayed linear attention S_t = lam_h S_(t-1) + k_t v_t^T,
// o_t = S_t^T q_t with the state in fp32 registers. A workgroup owns a
// 64-column slice of one (sequence, head) state — columns evolve
// independently, which gives Dv/64-way parallelism per head on top of
// sequences x heads — and walks the chunk's tokens in order.
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

constexpr int LA_WAVES = 4;   // heads per workgroup
constexpr int LA_KEYS = 4;    // keys per online-softmax update

template <typename T, int DPL>
__global__ void __launch_bounds__(LA_WAVES * WAVE)
latent_attn_kernel(const T* __restrict__ q_abs,   // [H, Tn, C]
                   const T* __restrict__ q_rot, long qr_tok, long qr_head,
                   const T* __restrict__ gate, long gate_tok,
                   const T* __restrict__ cache,   // [blocks, bs, C + R]
                   const int* __restrict__ block_table, int bt_stride,
                   const int* __restrict__ positions,
                   const int* __restrict__ seq_idx,
                   T* __restrict__ out,           // [H, Tn, C]
                   float* __restrict__ part_acc,  // [splits, H, Tn, C]
                   float* __restrict__ part_ml,   // [splits, H, Tn, 2]
                   int Tn, int H, int C, int R, int bs, int window,
                   float scale, const float* __restrict__ sink) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x % WAVE;
    const int h = blockIdx.y * LA_WAVES + threadIdx.x / WAVE;
    if (h >= H) return;
    const int Dk = C + R;
    const int p = positions[t];
    const int* bt = block_table + (long)seq_idx[t] * bt_stride;
    int lo = max(0, p - window + 1);
    int last = p;
    const int splits = gridDim.z;
    if (splits > 1) {
        // this workgroup's share of the visible keys (whole key groups)
        int per = (p - lo + splits) / splits;
        per = (per + LA_KEYS - 1) / LA_KEYS * LA_KEYS;
        lo += blockIdx.z * per;
        last = min(p, lo + per - 1);
    }

    float qv[DPL], acc[DPL];
    const T* qa = q_abs + ((long)h * Tn + t) * C;
    const T* qr = q_rot + (long)t * qr_tok + (long)h * qr_head;
#pragma unroll
    for (int j = 0; j < DPL; ++j) {
        const int c = lane + WAVE * j;
        float v = 0.f;
        if (c < C) v = ldf(qa + c);
        else if (c < Dk) v = ldf(qr + (c - C));
        qv[j] = v * scale;
        acc[j] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    for (int key = lo; key <= last; key += LA_KEYS) {
        float kv[LA_KEYS][DPL], s[LA_KEYS];
#pragma unroll
        for (int u = 0; u < LA_KEYS; ++u) {
            const int kp = min(key + u, last);  // clamp: stay inside the pages
            const T* row = cache + ((long)bt[kp / bs] * bs + kp % bs) * Dk;
            float d = 0.f;
#pragma unroll
            for (int j = 0; j < DPL; ++j) {
                const int c = lane + WAVE * j;
                kv[u][j] = c < Dk ? ldf(row + c) : 0.f;
                d += qv[j] * kv[u][j];
            }
            s[u] = d;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
#pragma unroll
            for (int u = 0; u < LA_KEYS; ++u) s[u] += __shfl_xor(s[u], off);
        }
        float mn = m;
#pragma unroll
        for (int u = 0; u < LA_KEYS; ++u) {
            if (key + u > last) s[u] = -INFINITY;
            mn = fmaxf(mn, s[u]);
        }
        const float a = expf(m - mn);
        float pu[LA_KEYS], ps = 0.f;
#pragma unroll
        for (int u = 0; u < LA_KEYS; ++u) {
            pu[u] = expf(s[u] - mn);
            ps += pu[u];
        }
        l = l * a + ps;
#pragma unroll
        for (int j = 0; j < DPL; ++j) {
            float v = acc[j] * a;
#pragma unroll
            for (int u = 0; u < LA_KEYS; ++u) v += pu[u] * kv[u][j];
            acc[j] = v;
        }
        m = mn;
    }
    if (splits > 1) {
        // unnormalized partial + (max, sum); an empty share leaves l = 0
        const long row = ((long)blockIdx.z * H + h) * Tn + t;
#pragma unroll
        for (int j = 0; j < DPL; ++j) {
            const int c = lane + WAVE * j;
            if (c < C) part_acc[row * C + c] = acc[j];
        }
        if (lane == 0) {
            part_ml[row * 2] = m;
            part_ml[row * 2 + 1] = l;
        }
        return;
    }
    const float g = 1.f / (1.f + expf(-ldf(gate + (long)t * gate_tok + h)));
    float r = g / l;
    if (sink) {
        // a logit that joins the denominator without key or value
        const float sk = sink[h];
        const float M = fmaxf(m, sk);
        const float w = expf(m - M);
        r = g * w / (l * w + expf(sk - M));
    }
    T* o = out + ((long)h * Tn + t) * C;
#pragma unroll
    for (int j = 0; j < DPL; ++j) {
        const int c = lane + WAVE * j;
        if (c < C) stf(o + c, acc[j] * r);
    }
}


// ------------------------------------------------- latent attention, MFMA
// bf16 prompt portions: workgroup = 16 consecutive queries of one sequence
// x 4 heads (one wave per head; all heads share the cached rows, so one
// staged key tile serves 64 query rows). Per 32-key tile: S = Q K^T on
// v_mfma_f32_16x16x32_bf16 (fp32 scores, scaled in fp32), window + causal
// mask, online softmax in fp32, then O += P K[:, :C] with the fp32 weights
// carried as a bf16 pair (hi + lo, two MFMAs) so they keep ~16 mantissa
// bits. Fragment maps (gfx950): A 16x32: lane -> row l&15, k (l>>4)*8+e;
// B 32x16: lane -> col l&15, k (l>>4)*8+e; C 16x16: col l&15, rows
// (l>>4)*4+r.
constexpr int LM_TN = 32;
constexpr int LM_PAD = 8;

template <int KSTEPS, bool DECODE>
__global__ void __launch_bounds__(256)
latent_attn_mfma_kernel(const unsigned short* __restrict__ q_abs,
                        const unsigned short* __restrict__ q_rot, long qr_tok,
                        long qr_head, const unsigned short* __restrict__ gate,
                        long gate_tok,
                        const unsigned short* __restrict__ cache,
                        const int* __restrict__ block_table, int bt_stride,
                        const int* __restrict__ cu,
                        const int* __restrict__ positions,
                        const int* __restrict__ seq_idx,
                        unsigned short* __restrict__ out,
                        float* __restrict__ part_acc,
                        float* __restrict__ part_ml, int Tn, int H, int C,
                        int R, int bs, int window, float scale,
                        const float* __restrict__ sink) {
    constexpr int DKP = KSTEPS * 32;
    constexpr int KS = DKP + LM_PAD;       // key tile row stride
    constexpr int PS = LM_TN + LM_PAD;     // weight tile row stride
    __shared__ __attribute__((aligned(16))) unsigned short k_s[LM_TN * KS];
    __shared__ __attribute__((aligned(16))) unsigned short p_hi[64 * PS];
    __shared__ __attribute__((aligned(16))) unsigned short p_lo[64 * PS];

    // PREFILL: rows = 16 queries of sequence blockIdx.z, wave = head.
    // DECODE:  rows = 16 heads of token blockIdx.x, the token's visible keys
    //          split over blockIdx.z. The four waves stage the key tile
    //          together, each recomputes the (small) score tile, and each
    //          accumulates every fourth 16-column block of the output.
    constexpr int NTH = 256;
    constexpr int NBW = DECODE ? (KSTEPS * 2 + 3) / 4 : KSTEPS * 2;
    const int seq = DECODE ? seq_idx[blockIdx.x] : (int)blockIdx.z;
    const int s0 = DECODE ? (int)blockIdx.x : cu[seq];
    const int QL = DECODE ? 1 : cu[seq + 1] - s0;
    const int q0 = DECODE ? 0 : blockIdx.x * 16;
    if (q0 >= QL) return;
    const int tid = threadIdx.x, lane = tid % WAVE, wid = tid / WAVE;
    const int lg = lane >> 4, li = lane & 15;
    // head of this lane's A row (li) / of the wave
    const int h = DECODE ? blockIdx.y * 16 + li : blockIdx.y * 4 + wid;
    const bool head_ok = h < H;
    const int Dk = C + R;
    const int hist = positions[s0];
    const int* bt = block_table + (long)seq * bt_stride;

    bf16x8 a_q[KSTEPS];
    {
        const int row = DECODE ? 0 : q0 + li;
        const bool ok = head_ok && row < QL;
        const unsigned short* qa = q_abs + ((long)h * Tn + s0 + row) * C;
        const unsigned short* qr = q_rot + (long)(s0 + row) * qr_tok +
                                   (long)h * qr_head;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const int c0 = ks * 32 + lg * 8;
            short8 raw = {0, 0, 0, 0, 0, 0, 0, 0};
            if (ok && c0 + 8 <= C) {
                // C is a multiple of 8 here: the unit lies inside the
                // (16 B aligned) absorbed-query row
                raw = *reinterpret_cast<const short8*>(qa + c0);
            } else if (ok && c0 < Dk) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    raw[e] = (short)qr[c0 + e - C];
            }
            a_q[ks] = __builtin_bit_cast(bf16x8, raw);
        }
    }
    float m_run[4], l_run[4];
    f32x4 o_acc[NBW];
#pragma unroll
    for (int r = 0; r < 4; ++r) { m_run[r] = -1e30f; l_run[r] = 0.f; }
#pragma unroll
    for (int j = 0; j < NBW; ++j) o_acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int last_row = min(q0 + 15, QL - 1);
    int kv_lo = max(0, hist + q0 - window + 1);
    int kv_end = hist + last_row + 1;
    if (DECODE && gridDim.z > 1) {
        int per = (kv_end - kv_lo + (int)gridDim.z - 1) / (int)gridDim.z;
        per = (per + LM_TN - 1) / LM_TN * LM_TN;
        kv_lo += blockIdx.z * per;
        kv_end = min(kv_end, kv_lo + per);
    }

    for (int kb = kv_lo; kb < kv_end; kb += LM_TN) {
        __syncthreads();   // previous tile's reads of k_s are done
        constexpr int UNITS = DKP / 8;
        for (int i = tid; i < LM_TN * UNITS; i += NTH) {
            const int key = i / UNITS, d = (i - key * UNITS) * 8;
            const int gk = kb + key;
            short8 raw = {0, 0, 0, 0, 0, 0, 0, 0};
            if (gk < kv_end && d < Dk)
                raw = *reinterpret_cast<const short8*>(
                    cache + ((long)bt[gk / bs] * bs + gk % bs) * Dk + d);
            *reinterpret_cast<short8*>(k_s + key * KS + d) = raw;
        }
        __syncthreads();

        f32x4 sfrag[LM_TN / 16];
#pragma unroll
        for (int f = 0; f < LM_TN / 16; ++f) {
            f32x4 acc{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                const bf16x8 bk = *reinterpret_cast<const bf16x8*>(
                    k_s + (f * 16 + li) * KS + ks * 32 + lg * 8);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_q[ks], bk, acc,
                                                              0, 0, 0);
            }
            sfrag[f] = acc;
        }
        float pmax[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) pmax[r] = -1e30f;
#pragma unroll
        for (int f = 0; f < LM_TN / 16; ++f) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // DECODE: every row is the same token (rows are heads)
                const int qrow = DECODE ? 0 : q0 + lg * 4 + r;
                const int key = kb + f * 16 + li;
                const int back = hist + qrow - key;
                const bool vis = qrow < QL && back >= 0 && back < window &&
                                 key < kv_end;
                sfrag[f][r] = vis ? sfrag[f][r] * scale : -1e30f;
                pmax[r] = fmaxf(pmax[r], sfrag[f][r]);
            }
        }
#pragma unroll
        for (int off = 1; off < 16; off <<= 1)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                pmax[r] = fmaxf(pmax[r], __shfl_xor(pmax[r], off));
        float alpha[4], psum[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float mn = fmaxf(m_run[r], pmax[r]);
            alpha[r] = expf(m_run[r] - mn);
            m_run[r] = mn;
            psum[r] = 0.f;
        }
#pragma unroll
        for (int f = 0; f < LM_TN / 16; ++f) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float pv = expf(sfrag[f][r] - m_run[r]);
                if (sfrag[f][r] <= -1e29f) pv = 0.f;
                psum[r] += pv;
                const unsigned short hi = f2bf(pv);
                const int at = (wid * 16 + lg * 4 + r) * PS + f * 16 + li;
                p_hi[at] = hi;
                p_lo[at] = f2bf(pv - bf2f(hi));
            }
        }
#pragma unroll
        for (int off = 1; off < 16; off <<= 1)
#pragma unroll
            for (int r = 0; r < 4; ++r) psum[r] += __shfl_xor(psum[r], off);
#pragma unroll
        for (int r = 0; r < 4; ++r) l_run[r] = l_run[r] * alpha[r] + psum[r];
#pragma unroll
        for (int j = 0; j < NBW; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) o_acc[j][r] *= alpha[r];
        __syncthreads();   // weight tile visible to the wave's other lanes
        const bf16x8 a_hi = *reinterpret_cast<const bf16x8*>(
            p_hi + (wid * 16 + li) * PS + lg * 8);
        const bf16x8 a_lo = *reinterpret_cast<const bf16x8*>(
            p_lo + (wid * 16 + li) * PS + lg * 8);
#pragma unroll
        for (int j = 0; j < NBW; ++j) {
            const int nb = DECODE ? j * 4 + wid : j;
            if (nb * 16 < C) {
                short8 raw;
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    raw[e] = (short)k_s[(lg * 8 + e) * KS + nb * 16 + li];
                const bf16x8 bv = __builtin_bit_cast(bf16x8, raw);
                o_acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    a_hi, bv, o_acc[j], 0, 0, 0);
                o_acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    a_lo, bv, o_acc[j], 0, 0, 0);
            }
        }
    }
    if (DECODE) {
        // C layout: this lane holds heads (rows) lg*4 + r, column li
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int hh = blockIdx.y * 16 + lg * 4 + r;
            if (hh >= H) continue;
            if (gridDim.z > 1) {
                const long row = ((long)blockIdx.z * H + hh) * Tn + s0;
#pragma unroll
                for (int j = 0; j < NBW; ++j) {
                    const int c = (j * 4 + wid) * 16 + li;
                    if (c < C) part_acc[row * C + c] = o_acc[j][r];
                }
                if (li == 0 && wid == 0) {
                    part_ml[row * 2] = m_run[r];
                    part_ml[row * 2 + 1] = l_run[r];
                }
            } else {
                const float g = 1.f / (1.f + expf(-bf2f(
                    gate[(long)s0 * gate_tok + hh])));
                float inv = l_run[r] > 0.f ? g / l_run[r] : 0.f;
                if (sink) {
                    const float sk = sink[hh];
                    const float M = fmaxf(m_run[r], sk);
                    const float w = expf(m_run[r] - M);
                    inv = g * w / (l_run[r] * w + expf(sk - M));
                }
                unsigned short* orow = out + ((long)hh * Tn + s0) * C;
#pragma unroll
                for (int j = 0; j < NBW; ++j) {
                    const int c = (j * 4 + wid) * 16 + li;
                    if (c < C) orow[c] = f2bf(o_acc[j][r] * inv);
                }
            }
        }
        return;
    }
    if (!head_ok) return;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int qrow = q0 + lg * 4 + r;
        if (qrow >= QL) continue;
        const float g = 1.f / (1.f + expf(-bf2f(
            gate[(long)(s0 + qrow) * gate_tok + h])));
        float inv = l_run[r] > 0.f ? g / l_run[r] : 0.f;
        if (sink) {
            const float sk = sink[h];
            const float M = fmaxf(m_run[r], sk);
            const float w = expf(m_run[r] - M);
            inv = g * w / (l_run[r] * w + expf(sk - M));
        }
        unsigned short* orow = out + ((long)h * Tn + s0 + qrow) * C;
#pragma unroll
        for (int j = 0; j < NBW; ++j) {
            const int c = j * 16 + li;
            if (c < C) orow[c] = f2bf(o_acc[j][r] * inv);
        }
    }
}

// merge the key-split partials of one (token, head): one workgroup per row.
// In every wave, lane z < splits holds share z's (max, sum); the merge
// weights exp(m_z - M) are computed once per wave and broadcast by shuffle,
// and each thread merges its columns with `splits` independent loads.
constexpr int LC_THREADS = 256;

template <typename T>
__global__ void __launch_bounds__(LC_THREADS)
latent_attn_combine_kernel(const float* __restrict__ part_acc,
                           const float* __restrict__ part_ml,
                           const T* __restrict__ gate, long gate_tok,
                           T* __restrict__ out, int splits, int Tn, int H,
                           int C, const float* __restrict__ sink) {
    const int t = blockIdx.x, h = blockIdx.y;
    const int lane = threadIdx.x % WAVE;
    float m = -INFINITY, l = 0.f;
    if (lane < splits) {
        const long row = ((long)lane * H + h) * Tn + t;
        m = part_ml[row * 2];
        l = part_ml[row * 2 + 1];
    }
    float M = wave_max(l > 0.f ? m : -INFINITY);
    if (sink) M = fmaxf(M, sink[h]);
    const float w = l > 0.f ? expf(m - M) : 0.f;
    float L = wave_sum(l * w);
    if (sink) L += expf(sink[h] - M);
    const float g = 1.f / (1.f + expf(-ldf(gate + (long)t * gate_tok + h)));
    const float r = g / L;
    T* o = out + ((long)h * Tn + t) * C;
    // uniform trip count: every lane takes part in every shuffle
    for (int c0 = 0; c0 < C; c0 += LC_THREADS) {
        const int c = c0 + threadIdx.x;
        float a = 0.f;
        for (int z = 0; z < splits; ++z) {
            const float wz = __shfl(w, z);
            if (c < C)
                a += part_acc[(((long)z * H + h) * Tn + t) * C + c] * wz;
        }
        if (c < C) stf(o + c, a * r);
    }
}

// ------------------------------------------------------------- lightning
constexpr int LI_COLS = 64;    // state columns per workgroup (one per lane)
constexpr int LI_GROUPS = 4;   // row groups = waves; each owns D/4 state rows
constexpr int LI_TB = 8;       // tokens staged per round

DEV_INLINE float silu_f(float x) { return x / (1.f + expf(-x)); }

// Workgroup = (sequence, head, 64-column slice of the state). Thread
// (g, col) keeps rows [g*DPT, (g+1)*DPT) of column col in registers. Per
// round of LI_TB tokens the block stages silu(q), silu(k) (all D rows) and
// silu(v) (its columns) in LDS once — wave g then reads q/k as broadcasts —
// and the four row groups' partial outputs are summed through LDS.
//
// MODE 0: a whole chunk per workgroup, from the sequence's carried state.
// Long chunks are cut into LI_SEG-token segments that run in parallel:
// MODE 1: a segment from a ZERO state; local outputs to `out`, the
//         segment's final local state to the workspace `ws`;
//   (lightning_scan_kernel then turns ws into the true state at each
//    segment's start and writes the sequence's final state to its slot)
// MODE 2: adds lam^(i+1) * S_start^T q_i to the segment's outputs (state
//         fixed, no update), i = token index within the segment.
// S_t = lam^(i+1) S_start + S_local,t, so modes 1+2 equal mode 0 up to fp32
// summation order.
constexpr int LI_SEG = 256;

// segment index -> (sequence, first row, end row); false when out of range
DEV_INLINE bool li_segment(const int* __restrict__ cu, int B, int seg,
                           int* b_out, int* lo, int* hi) {
    int first = 0;
    for (int b = 0; b < B; ++b) {
        const int len = cu[b + 1] - cu[b];
        const int n = (len + LI_SEG - 1) / LI_SEG;
        if (seg < first + n) {
            *b_out = b;
            *lo = cu[b] + (seg - first) * LI_SEG;
            *hi = min(cu[b + 1], *lo + LI_SEG);
            return true;
        }
        first += n;
    }
    return false;
}

//
// FORM 0 (lightning): q, k, v enter as silu of the projections.
// FORM 1 (retention): q and k are rotated by position — coordinate i of the
// first `rdims` pairs with i + rdims/2, angle from the fp32 cos/sin tables
// [max_pos, rdims/2] — k is also multiplied by k_scale, v enters as is.
template <typename T, int FORM>
DEV_INLINE float li_load_qk(const T* __restrict__ row, int d, int rdims,
                            const float* __restrict__ cs,
                            const float* __restrict__ sn) {
    const float x = ldf(row + d);
    if (FORM == 0) return silu_f(x);
    if (d >= rdims) return x;
    const int half = rdims / 2;
    const int j = d < half ? d : d - half;
    const float y = ldf(row + (d < half ? d + half : d - half));
    return d < half ? x * cs[j] - y * sn[j] : x * cs[j] + y * sn[j];
}

template <typename T, int DPT, int MODE, int FORM>
__global__ void __launch_bounds__(LI_COLS * LI_GROUPS)
lightning_kernel(const T* __restrict__ q, const T* __restrict__ k,
                 const T* __restrict__ v, long tok_stride,
                 const float* __restrict__ cos_t,
                 const float* __restrict__ sin_t, int rdims, float k_scale,
                 const float* __restrict__ decay,
                 float* __restrict__ state,        // [slots, H, D, Dv]
                 const int* __restrict__ state_slots,
                 const int* __restrict__ cu,
                 const int* __restrict__ positions,
                 float* __restrict__ out,          // [Tn, H * Dv]
                 float* __restrict__ ws,           // [segments, H, D, Dv]
                 int B, int H, int D, int Dv) {
    constexpr int DMAX = DPT * LI_GROUPS;
    __shared__ float qs[LI_TB][DMAX];
    __shared__ float ks[LI_TB][DMAX];
    __shared__ float vs[LI_TB][LI_COLS];
    __shared__ float red[LI_TB][LI_GROUPS][LI_COLS];
    const int h = blockIdx.y;
    int b, lo, hi;
    if (MODE == 0) {
        b = blockIdx.x;
        lo = cu[b];
        hi = cu[b + 1];
    } else if (!li_segment(cu, B, blockIdx.x, &b, &lo, &hi)) {
        return;
    }
    if (hi <= lo) return;
    const int nth = LI_COLS * LI_GROUPS;
    const int g = threadIdx.x / LI_COLS, col = threadIdx.x % LI_COLS;
    const int c0 = blockIdx.z * LI_COLS;
    const int dv = c0 + col;
    const bool live = dv < Dv;
    const int d0 = g * DPT;
    const float lam = decay[h];
    const float log_lam = logf(lam);
    float* st = MODE == 0
        ? state + (((long)state_slots[b] * H + h) * D) * Dv + dv
        : ws + (((long)blockIdx.x * H + h) * D) * Dv + dv;
    const bool fresh = MODE == 1 || (MODE == 0 && positions[lo] == 0);
    float s[DPT];
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
        const int d = d0 + i;
        s[i] = (!fresh && live && d < D) ? st[(long)d * Dv] : 0.f;
    }
    for (int t0 = lo; t0 < hi; t0 += LI_TB) {
        const int n = min(LI_TB, hi - t0);
        for (int idx = threadIdx.x; idx < n * DMAX; idx += nth) {
            const int tt = idx / DMAX, d = idx - tt * DMAX;
            const long base = (long)(t0 + tt) * tok_stride + (long)h * D;
            const float* cs = nullptr;
            const float* sn = nullptr;
            if (FORM == 1 && rdims > 0) {
                const long pr = (long)positions[t0 + tt] * (rdims / 2);
                cs = cos_t + pr;
                sn = sin_t + pr;
            }
            qs[tt][d] = d < D ? li_load_qk<T, FORM>(q + base, d, rdims, cs, sn)
                              : 0.f;
            if (MODE != 2)
                ks[tt][d] = d < D ? li_load_qk<T, FORM>(k + base, d, rdims, cs,
                                                        sn) * k_scale
                                  : 0.f;
        }
        if (MODE != 2) {
            for (int idx = threadIdx.x; idx < n * LI_COLS; idx += nth) {
                const int tt = idx / LI_COLS, c = idx - tt * LI_COLS;
                float vv = 0.f;
                if (c0 + c < Dv) {
                    vv = ldf(v + (long)(t0 + tt) * tok_stride + (long)h * Dv +
                             c0 + c);
                    if (FORM == 0) vv = silu_f(vv);
                }
                vs[tt][c] = vv;
            }
        }
        __syncthreads();
        for (int tt = 0; tt < n; ++tt) {
            float part = 0.f;
            if (MODE == 2) {
#pragma unroll
                for (int i = 0; i < DPT; ++i) part += s[i] * qs[tt][d0 + i];
            } else {
                const float vv = vs[tt][col];
#pragma unroll
                for (int i = 0; i < DPT; ++i) {
                    s[i] = lam * s[i] + ks[tt][d0 + i] * vv;
                    part += s[i] * qs[tt][d0 + i];
                }
            }
            red[tt][g][col] = part;
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < n * LI_COLS; idx += nth) {
            const int tt = idx / LI_COLS, c = idx - tt * LI_COLS;
            float o = 0.f;
#pragma unroll
            for (int gg = 0; gg < LI_GROUPS; ++gg) o += red[tt][gg][c];
            if (c0 + c < Dv) {
                float* op = out + (long)(t0 + tt) * H * Dv + (long)h * Dv +
                            c0 + c;
                if (MODE == 2)
                    *op += o * expf(log_lam * (float)(t0 + tt - lo + 1));
                else
                    *op = o;
            }
        }
    }
    if (MODE != 2 && live) {
#pragma unroll
        for (int i = 0; i < DPT; ++i) {
            const int d = d0 + i;
            if (d < D) st[(long)d * Dv] = s[i];
        }
    }
}

// Per (sequence, head), one thread per state element: walk the sequence's
// segments in order, replacing each segment's local final state in ws by
// the true state at that segment's start, and leave the sequence's final
// state in its slot.
__global__ void lightning_scan_kernel(const float* __restrict__ decay,
                                      float* __restrict__ state,
                                      const int* __restrict__ state_slots,
                                      const int* __restrict__ cu,
                                      const int* __restrict__ positions,
                                      float* __restrict__ ws, int H,
                                      int DDv) {
    const int b = blockIdx.x, h = blockIdx.y;
    const int e = blockIdx.z * blockDim.x + threadIdx.x;
    if (e >= DDv) return;
    const int lo = cu[b], len = cu[b + 1] - lo;
    if (len <= 0) return;
    int first = 0;
    for (int bb = 0; bb < b; ++bb)
        first += (cu[bb + 1] - cu[bb] + LI_SEG - 1) / LI_SEG;
    const float log_lam = logf(decay[h]);
    float* slot = state + ((long)state_slots[b] * H + h) * DDv + e;
    float S = positions[lo] == 0 ? 0.f : *slot;
    const int nseg = (len + LI_SEG - 1) / LI_SEG;
    for (int sg = 0; sg < nseg; ++sg) {
        float* w = ws + ((long)(first + sg) * H + h) * DDv + e;
        const float local = *w;
        *w = S;
        const int n = min(LI_SEG, len - sg * LI_SEG);
        S = expf(log_lam * (float)n) * S + local;
    }
    *slot = S;
}

// ------------------------------------------------------------ delta rule
// Gated delta rule on a memory M (key rows x value columns), fp32, per
// token:  M <- g * M;  delta = beta (v - M^T k);  M <- M + k delta^T;
// y = M^T q.  Since y = (gM)^T q + delta (k . q), both sums over the key
// axis run on the faded memory in ONE pass.
// A workgroup is ONE wave that owns 64/RG columns of one (sequence, value
// head) state: lane (c, r) = (lane / RG, lane % RG) keeps rows
// [r*DPT, (r+1)*DPT) of column c in registers. The RG row groups are
// neighbouring lanes, so the two sums over the key axis are DPP adds inside
// a row of 16 lanes (no LDS round trip), and nothing but the staging of
// DR_TB tokens' q/k/g/v/beta through LDS needs a barrier. Columns evolve
// independently -> sequences x heads x Dv*RG/64 waves; the launcher picks
// RG = 4 when sequences x heads alone fill the chip (decode: 64-byte state
// rows per group) and 8 or 16 for a few long prompt portions. Tokens are
// walked in order (token t reads the state token t-1 left).
constexpr int DR_TB = 8;

template <int CTRL> DEV_INLINE float dr_dpp_add(float x) {
    const int y = __builtin_amdgcn_update_dpp(
        0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true);
    return x + __builtin_bit_cast(float, y);
}
// sum over the RG neighbouring lanes of a group; every lane gets the total
template <int RG> DEV_INLINE float dr_group_sum(float x) {
    x = dr_dpp_add<0xB1>(x);                  // quad_perm [1,0,3,2]
    x = dr_dpp_add<0x4E>(x);                  // quad_perm [2,3,0,1]
    if (RG >= 8) x = dr_dpp_add<0x141>(x);    // row_half_mirror
    if (RG >= 16) x = dr_dpp_add<0x140>(x);   // row_mirror
    return x;
}

template <int DPT, int RG, bool CHDEC>
__global__ void __launch_bounds__(WAVE)
delta_rule_kernel(const float* __restrict__ q, const float* __restrict__ k,
                  long qk_tok, const float* __restrict__ v, long v_tok,
                  const float* __restrict__ beta,   // [Tn, H]
                  const float* __restrict__ g,      // [Tn, H] | [Tn, H, D]
                  float* __restrict__ state,        // [slots, H, D, Dv]
                  const int* __restrict__ state_slots,
                  const int* __restrict__ cu,
                  const int* __restrict__ positions,
                  float* __restrict__ out,          // [Tn, H, Dv]
                  int H, int G, int D, int Dv) {
    static_assert(DPT % 4 == 0, "16-byte LDS reads");
    constexpr int DMAX = DPT * RG;
    constexpr int CW = WAVE / RG;
    __shared__ __attribute__((aligned(16))) float qs[DR_TB][DMAX];
    __shared__ __attribute__((aligned(16))) float ks[DR_TB][DMAX];
    __shared__ __attribute__((aligned(16))) float gs[DR_TB][CHDEC ? DMAX : 4];
    __shared__ float vs[DR_TB][CW];
    __shared__ float bs[DR_TB];
    __shared__ float kqs[DR_TB];
    const int b = blockIdx.x, h = blockIdx.y;
    const int lo = cu[b], hi = cu[b + 1];
    if (hi <= lo) return;
    const int lane = threadIdx.x;
    const int c = lane / RG, r = lane % RG;
    const int c0 = blockIdx.z * CW;
    const int dv = c0 + c;
    const bool live = dv < Dv;
    const int d0 = r * DPT;
    const int kvh = h / (H / G);
    float* st = state + (((long)state_slots[b] * H + h) * D) * Dv + dv;
    const bool fresh = positions[lo] == 0;
    float s[DPT];
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
        const int d = d0 + i;
        s[i] = (!fresh && live && d < D) ? st[(long)d * Dv] : 0.f;
    }
    // The next DR_TB tokens' inputs are fetched into registers while the
    // current ones are consumed from LDS, so HBM latency stays off the
    // token-serial chain.
    constexpr int PQ = (DR_TB * DMAX + WAVE - 1) / WAVE;
    constexpr int PV = (DR_TB * CW + WAVE - 1) / WAVE;
    float pq[PQ], pk[PQ], pg[CHDEC ? PQ : 1], pv[PV], pb = 0.f;
    auto fetch = [&](int t0) {
        const int n = min(DR_TB, hi - t0);
#pragma unroll
        for (int e = 0; e < PQ; ++e) {
            const int idx = lane + e * WAVE;
            const int tt = idx / DMAX, d = idx - tt * DMAX;
            const bool ok = tt < n && d < D;
            const long base = (long)(t0 + tt) * qk_tok + (long)kvh * D + d;
            pq[e] = ok ? q[base] : 0.f;
            pk[e] = ok ? k[base] : 0.f;
            if (CHDEC)
                pg[e] = ok ? g[((long)(t0 + tt) * H + h) * D + d] : 1.f;
        }
#pragma unroll
        for (int e = 0; e < PV; ++e) {
            const int idx = lane + e * WAVE;
            const int tt = idx / CW, cc = idx - tt * CW;
            pv[e] = (tt < n && c0 + cc < Dv)
                ? v[(long)(t0 + tt) * v_tok + (long)h * Dv + c0 + cc] : 0.f;
        }
        if (lane < n) {
            pb = beta[(long)(t0 + lane) * H + h];
            if (!CHDEC) pg[0] = g[(long)(t0 + lane) * H + h];
        }
    };
    fetch(lo);
    for (int t0 = lo; t0 < hi; t0 += DR_TB) {
        const int n = min(DR_TB, hi - t0);
#pragma unroll
        for (int e = 0; e < PQ; ++e) {
            const int idx = lane + e * WAVE;
            if (idx < DR_TB * DMAX) {
                (&qs[0][0])[idx] = pq[e];
                (&ks[0][0])[idx] = pk[e];
                if (CHDEC) (&gs[0][0])[idx] = pg[e];
            }
        }
#pragma unroll
        for (int e = 0; e < PV; ++e) {
            const int idx = lane + e * WAVE;
            if (idx < DR_TB * CW) (&vs[0][0])[idx] = pv[e];
        }
        if (lane < n) {
            bs[lane] = pb;
            if (!CHDEC) gs[lane][0] = pg[0];
        }
        __syncthreads();
        if (t0 + DR_TB < hi) fetch(t0 + DR_TB);
        // k . q of each staged token, once (it does not involve the state):
        // 8 neighbouring lanes per token
        {
            const int tt = lane / 8, part = lane % 8;
            float a = 0.f;
            for (int d = part; d < DMAX; d += 8) a += ks[tt][d] * qs[tt][d];
            a = dr_group_sum<8>(a);
            if (part == 0) kqs[tt] = a;
        }
        __syncthreads();
        for (int tt = 0; tt < n; ++tt) {
            // this lane's slice of k, q (and the per-channel decay) into
            // registers with 16-byte LDS reads; k is used twice
            float kr[DPT], qr[DPT], gr[CHDEC ? DPT : 1];
#pragma unroll
            for (int i = 0; i < DPT; i += 4) {
                const f32x4 a =
                    *reinterpret_cast<const f32x4*>(&ks[tt][d0 + i]);
                const f32x4 e =
                    *reinterpret_cast<const f32x4*>(&qs[tt][d0 + i]);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    kr[i + j] = a[j];
                    qr[i + j] = e[j];
                }
                if constexpr (CHDEC) {
                    const f32x4 w =
                        *reinterpret_cast<const f32x4*>(&gs[tt][d0 + i]);
#pragma unroll
                    for (int j = 0; j < 4; ++j) gr[i + j] = w[j];
                }
            }
            if constexpr (!CHDEC) gr[0] = gs[tt][0];
            float ka = 0.f, kb = 0.f, qa = 0.f, qb = 0.f;
#pragma unroll
            for (int i = 0; i < DPT; i += 2) {
                const float s0 = s[i] * gr[CHDEC ? i : 0];
                const float s1 = s[i + 1] * gr[CHDEC ? i + 1 : 0];
                s[i] = s0;
                s[i + 1] = s1;
                ka += kr[i] * s0;
                kb += kr[i + 1] * s1;
                qa += qr[i] * s0;
                qb += qr[i + 1] * s1;
            }
            const float kS = dr_group_sum<RG>(ka + kb);
            const float qS = dr_group_sum<RG>(qa + qb);
            const float u = bs[tt] * (vs[tt][c] - kS);
#pragma unroll
            for (int i = 0; i < DPT; ++i) s[i] += kr[i] * u;
            if (r == 0 && live)
                out[((long)(t0 + tt) * H + h) * Dv + dv] = qS + u * kqs[tt];
        }
        __syncthreads();
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < DPT; ++i) {
            const int d = d0 + i;
            if (d < D) st[(long)d * Dv] = s[i];
        }
    }
}

// ------------------------------------------------ attention with a sink
// Causal grouped-query softmax attention over paged keys/values
// [n_blocks, G, bs, D|Dv], any head size up to SA_MAXD, bf16 or fp32 pages.
// One wave per (token, up to 4 query heads of one key group, key split):
// tiles of 64 keys — for the scores a lane owns ONE key and walks its row
// against the queries held in LDS (fp32), the tile's max/sum are wave
// reductions, and for the weighted value sum lanes own output coordinates
// while the weights are read lane by lane. Scores, weights and accumulators are fp32; every score
// multiplier is already in q. The softmax denominator also counts
// exp(sink[h]) once when sink is given. Row t at position p sees cached
// positions j <= p (j > p - window when window > 0). With gridDim.z > 1
// each split writes its (max, sum, partial) and sink_attn_combine merges.
constexpr int SA_WAVES = 4;
constexpr int SA_MAXD = 256;

// scores of one key row against REP query vectors held in LDS (fp32).
// The row is fetched in blocks of SA_BLK 16-byte loads that are all issued
// before any is consumed: a rolled loop of load -> use would pay one memory
// latency per 16 bytes.
constexpr int SA_BLK = 8;

template <int REP>
DEV_INLINE void sa_dots_f32(const float* __restrict__ kr,
                            const float* __restrict__ qv, int D,
                            float* __restrict__ sc) {
    int d = 0;
    if (D % 4 == 0) {
        for (; d + 4 * SA_BLK <= D; d += 4 * SA_BLK) {
            f32x4 x[SA_BLK];
#pragma unroll
            for (int c = 0; c < SA_BLK; ++c)
                x[c] = *reinterpret_cast<const f32x4*>(kr + d + 4 * c);
#pragma unroll
            for (int c = 0; c < SA_BLK; ++c)
#pragma unroll
                for (int r = 0; r < REP; ++r) {
                    const float* qr = qv + r * D + d + 4 * c;
                    sc[r] += x[c][0] * qr[0] + x[c][1] * qr[1] +
                             x[c][2] * qr[2] + x[c][3] * qr[3];
                }
        }
        for (; d < D; d += 4) {
            const f32x4 x = *reinterpret_cast<const f32x4*>(kr + d);
#pragma unroll
            for (int r = 0; r < REP; ++r) {
                const float* qr = qv + r * D + d;
                sc[r] += x[0] * qr[0] + x[1] * qr[1] + x[2] * qr[2] +
                         x[3] * qr[3];
            }
        }
    } else {
        for (; d < D; ++d) {
            const float x = kr[d];
#pragma unroll
            for (int r = 0; r < REP; ++r) sc[r] += x * qv[r * D + d];
        }
    }
}
template <int REP>
DEV_INLINE void sa_dots_bf16(const unsigned short* __restrict__ kr,
                             const float* __restrict__ qv, int D,
                             float* __restrict__ sc) {
    int d = 0;
    if (D % 8 == 0) {
        for (; d + 8 * SA_BLK <= D; d += 8 * SA_BLK) {
            short8 raw[SA_BLK];
#pragma unroll
            for (int c = 0; c < SA_BLK; ++c)
                raw[c] = *reinterpret_cast<const short8*>(kr + d + 8 * c);
#pragma unroll
            for (int c = 0; c < SA_BLK; ++c) {
                float x[8];
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    x[j] = bf2f((unsigned short)raw[c][j]);
#pragma unroll
                for (int r = 0; r < REP; ++r) {
                    const float* qr = qv + r * D + d + 8 * c;
                    float a = 0.f, b = 0.f;
#pragma unroll
                    for (int j = 0; j < 8; j += 2) {
                        a += x[j] * qr[j];
                        b += x[j + 1] * qr[j + 1];
                    }
                    sc[r] += a + b;
                }
            }
        }
        for (; d < D; d += 8) {
            float x[8];
            load_bf16x8(kr + d, x);
#pragma unroll
            for (int r = 0; r < REP; ++r) {
                const float* qr = qv + r * D + d;
                float a = 0.f, b = 0.f;
#pragma unroll
                for (int j = 0; j < 8; j += 2) {
                    a += x[j] * qr[j];
                    b += x[j + 1] * qr[j + 1];
                }
                sc[r] += a + b;
            }
        }
    } else {
        for (; d < D; ++d) {
            const float x = bf2f(kr[d]);
#pragma unroll
            for (int r = 0; r < REP; ++r) sc[r] += x * qv[r * D + d];
        }
    }
}
template <typename T, int REP> struct SaDots;
template <int REP> struct SaDots<float, REP> {
    static DEV_INLINE void run(const float* kr, const float* qv, int D,
                               float* sc) { sa_dots_f32<REP>(kr, qv, D, sc); }
};
template <int REP> struct SaDots<unsigned short, REP> {
    static DEV_INLINE void run(const unsigned short* kr, const float* qv,
                               int D, float* sc) {
        sa_dots_bf16<REP>(kr, qv, D, sc);
    }
};

// A wave serves REP query heads that share one key/value head (REP divides
// the group size), so each cached row is read once for all of them.
constexpr int SA_PV = 8;      // value rows in flight per step

// Output coordinate i of a lane. PAIR (even value size): a lane owns
// neighbouring coordinates 2*lane, 2*lane+1 (+128 per further pair) and
// fetches both with one load; otherwise lane, lane+64, ...
template <bool PAIR> DEV_INLINE int sa_coord(int lane, int i) {
    return PAIR ? (i >> 1) * (2 * WAVE) + 2 * lane + (i & 1) : lane + i * WAVE;
}
DEV_INLINE void sa_ld2(const float* p, float& a, float& b) {
    const float2v w = *reinterpret_cast<const float2v*>(p);
    a = w[0];
    b = w[1];
}
DEV_INLINE void sa_ld2(const unsigned short* p, float& a, float& b) {
    const unsigned int w = *reinterpret_cast<const unsigned int*>(p);
    a = bf2f((unsigned short)(w & 0xffffu));
    b = bf2f((unsigned short)(w >> 16));
}

template <typename T, int DPL, int REP, bool PAIR>
__global__ void __launch_bounds__(SA_WAVES * WAVE)
sink_attn_kernel(const T* __restrict__ q, long q_tok,
                 const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                 const int* __restrict__ block_table, int bt_stride,
                 const int* __restrict__ positions,
                 const int* __restrict__ seq_idx,
                 const float* __restrict__ sink, T* __restrict__ out,
                 long out_tok, float out_scale, float* __restrict__ part_acc,
                 float* __restrict__ part_ml, int Tn, int H, int G, int D,
                 int Dv, int bs, int window,
                 const T* __restrict__ head_gate, long hg_tok) {
    extern __shared__ __attribute__((aligned(16))) float sa_q[];
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int t = blockIdx.x;
    const int unit = blockIdx.y * SA_WAVES + wid;   // REP consecutive heads
    if (unit * REP >= H) return;      // no workgroup barrier below
    const int h0 = unit * REP;
    const int split = blockIdx.z, nsplit = gridDim.z;
    const int p = positions[t];
    const int g = h0 / (H / G);
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    // a split takes whole 64-key tiles, so no wave pays a full score pass
    // for a few keys; splits past the end stay empty (sum 0) for the merge
    const int per =
        ((p + 1 - lo + nsplit - 1) / nsplit + WAVE - 1) / WAVE * WAVE;
    const int klo = lo + split * per, khi = min(p + 1, klo + per);
    float* qv = sa_q + (long)wid * REP * D;
    for (int i = lane; i < REP * D; i += WAVE)
        qv[i] = ldf(q + (long)t * q_tok + (long)h0 * D + i);
    WAVE_LDS_SYNC();
    const int* bt = block_table + (long)seq_idx[t] * bt_stride;
    float m[REP], l[REP], acc[REP][DPL];
#pragma unroll
    for (int r = 0; r < REP; ++r) {
        m[r] = -INFINITY;
        l[r] = 0.f;
#pragma unroll
        for (int i = 0; i < DPL; ++i) acc[r][i] = 0.f;
    }
    for (int j0 = klo; j0 < khi; j0 += WAVE) {
        const int j = j0 + lane;
        const bool valid = j < khi;
        // lanes past the end point at the share's last key: a row this
        // sequence wrote (their weights are 0, and 0 x garbage is not 0)
        const int jc = min(j, khi - 1);
        const int row = (bt[jc / bs] * G + g) * bs + jc % bs;
        float sc[REP], pj[REP];
#pragma unroll
        for (int r = 0; r < REP; ++r) sc[r] = 0.f;
        const int nk = min(WAVE, khi - j0);
        if (valid) SaDots<T, REP>::run(k_cache + (long)row * D, qv, D, sc);
#pragma unroll
        for (int r = 0; r < REP; ++r) {
            const float s = valid ? sc[r] : -INFINITY;
            const float m_new = fmaxf(m[r], wave_max(s));
            pj[r] = valid ? expf(s - m_new) : 0.f;
            const float corr = expf(m[r] - m_new);
            l[r] = l[r] * corr + wave_sum(pj[r]);
#pragma unroll
            for (int i = 0; i < DPL; ++i) acc[r][i] *= corr;
            m[r] = m_new;
        }
#pragma unroll 2
        for (int jj = 0; jj < nk; jj += SA_PV) {
            float vv[SA_PV][DPL];
#pragma unroll
            for (int u = 0; u < SA_PV; ++u) {
                const T* vr =
                    v_cache + (long)__builtin_amdgcn_readlane(row, jj + u) * Dv;
                if constexpr (PAIR) {
#pragma unroll
                    for (int i = 0; i < DPL; i += 2) {
                        const int d = sa_coord<true>(lane, i);
                        vv[u][i] = vv[u][i + 1] = 0.f;
                        if (d < Dv) sa_ld2(vr + d, vv[u][i], vv[u][i + 1]);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < DPL; ++i) {
                        const int d = sa_coord<false>(lane, i);
                        vv[u][i] = d < Dv ? ldf(vr + d) : 0.f;
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < SA_PV; ++u)
#pragma unroll
                for (int r = 0; r < REP; ++r) {
                    // jj + u is wave-uniform: a scalar lane read, no LDS trip
                    const float pb = __builtin_bit_cast(
                        float, __builtin_amdgcn_readlane(
                                   __builtin_bit_cast(int, pj[r]), jj + u));
#pragma unroll
                    for (int i = 0; i < DPL; ++i) acc[r][i] += pb * vv[u][i];
                }
        }
    }
#pragma unroll
    for (int r = 0; r < REP; ++r) {
        const int h = h0 + r;
        if (nsplit == 1) {
            float L = l[r], w = 1.f;
            if (sink) {
                const float sk = sink[h];
                const float M = fmaxf(m[r], sk);
                w = expf(m[r] - M);
                L = l[r] * w + expf(sk - M);
            }
            float rcp = L > 0.f ? out_scale * w / L : 0.f;
            if (head_gate)      // sigmoid gate, one number per (token, head)
                rcp /= 1.f + expf(-ldf(head_gate + (long)t * hg_tok + h));
            T* o = out + (long)t * out_tok + (long)h * Dv;
#pragma unroll
            for (int i = 0; i < DPL; ++i) {
                const int d = sa_coord<PAIR>(lane, i);
                if (d < Dv) stf(o + d, acc[r][i] * rcp);
            }
        } else {
            const long prow = ((long)split * H + h) * Tn + t;
            if (lane == 0) {
                part_ml[prow * 2] = m[r];
                part_ml[prow * 2 + 1] = l[r];
            }
#pragma unroll
            for (int i = 0; i < DPL; ++i) {
                const int d = sa_coord<PAIR>(lane, i);
                if (d < Dv) part_acc[prow * Dv + d] = acc[r][i];
            }
        }
    }
}

// merge of the key splits: wave per (token, head)
template <typename T>
__global__ void __launch_bounds__(SA_WAVES * WAVE)
sink_attn_combine_kernel(const float* __restrict__ part_acc,
                         const float* __restrict__ part_ml,
                         const float* __restrict__ sink, T* __restrict__ out,
                         long out_tok, float out_scale, int splits, int Tn,
                         int H, int Dv, const T* __restrict__ head_gate,
                         long hg_tok) {
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int t = blockIdx.x, h = blockIdx.y * SA_WAVES + wid;
    if (h >= H) return;
    float m = -INFINITY, l = 0.f;
    if (lane < splits) {
        const long row = ((long)lane * H + h) * Tn + t;
        m = part_ml[row * 2];
        l = part_ml[row * 2 + 1];
    }
    float M = wave_max(l > 0.f ? m : -INFINITY);
    if (sink) M = fmaxf(M, sink[h]);
    const float w = l > 0.f ? expf(m - M) : 0.f;
    float L = wave_sum(l * w);
    if (sink) L += expf(sink[h] - M);
    float rcp = L > 0.f ? out_scale / L : 0.f;
    if (head_gate)
        rcp /= 1.f + expf(-ldf(head_gate + (long)t * hg_tok + h));
    T* o = out + (long)t * out_tok + (long)h * Dv;
    for (int d0 = 0; d0 < Dv; d0 += WAVE) {
        const int d = d0 + lane;
        const int dc = min(d, Dv - 1);      // clamped: every load is valid
        float a = 0.f;
        int z = 0;
        // four partial rows in flight per step
        for (; z + 4 <= splits; z += 4) {
            float x[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                x[u] = part_acc[(((long)(z + u) * H + h) * Tn + t) * Dv + dc];
#pragma unroll
            for (int u = 0; u < 4; ++u) a += x[u] * __shfl(w, z + u);
        }
        for (; z < splits; ++z)
            a += part_acc[(((long)z * H + h) * Tn + t) * Dv + dc] *
                 __shfl(w, z);
        if (d < Dv) stf(o + d, a * rcp);
    }
}

}  // namespace

#define LA_CASE(N)                                                            \
    case N:                                                                   \
        latent_attn_kernel<TT, N><<<grid, LA_WAVES * WAVE, 0, s>>>(           \
            (const TT*)q_abs, (const TT*)q_rot, qr_tok, qr_head,              \
            (const TT*)gate, gate_tok, (const TT*)cache, block_table,         \
            bt_stride, positions, seq_idx, (TT*)out, part_acc, part_ml, Tn,   \
            H, C, R, bs, window, scale, sink);                                \
        break;

template <typename TT>
static int latent_attn_dispatch(const void* q_abs, const void* q_rot,
                                long qr_tok, long qr_head, const void* gate,
                                long gate_tok, const void* cache,
                                const int* block_table, int bt_stride,
                                const int* positions, const int* seq_idx,
                                void* out, float* part_acc, float* part_ml,
                                int splits, int Tn, int H, int C, int R,
                                int bs, int window, float scale,
                                const float* sink, hipStream_t s) {
    const int need = (C + R + WAVE - 1) / WAVE;
    const int sizes[] = {1, 2, 3, 4, 6, 9, 12, 16};
    int dpl = 0;
    for (int z : sizes)
        if (z >= need) { dpl = z; break; }
    if (!dpl) return 1;
    const dim3 grid(Tn, (H + LA_WAVES - 1) / LA_WAVES, splits);
    switch (dpl) {
        LA_CASE(1) LA_CASE(2) LA_CASE(3) LA_CASE(4) LA_CASE(6) LA_CASE(9)
        LA_CASE(12) LA_CASE(16)
    }
    if (splits > 1) {
        const dim3 g2(Tn, H);
        latent_attn_combine_kernel<TT><<<g2, LC_THREADS, 0, s>>>(
            part_acc, part_ml, (const TT*)gate, gate_tok, (TT*)out, splits,
            Tn, H, C, sink);
    }
    return 0;
}

// returns nonzero when the row width (kv_rank + rot_dim) exceeds 1024
extern "C" int launch_latent_attn(const void* q_abs, const void* q_rot,
                                  long qr_tok, long qr_head, const void* gate,
                                  long gate_tok, const void* cache,
                                  const int* block_table, int bt_stride,
                                  const int* positions, const int* seq_idx,
                                  void* out, float* part_acc, float* part_ml,
                                  int splits, int Tn, int H, int C, int R,
                                  int bs, int window, float scale, int f32,
                                  const float* sink, hipStream_t s) {
    if (Tn == 0) return 0;
    if (f32)
        return latent_attn_dispatch<float>(
            q_abs, q_rot, qr_tok, qr_head, gate, gate_tok, cache, block_table,
            bt_stride, positions, seq_idx, out, part_acc, part_ml, splits, Tn,
            H, C, R, bs, window, scale, sink, s);
    return latent_attn_dispatch<unsigned short>(
        q_abs, q_rot, qr_tok, qr_head, gate, gate_tok, cache, block_table,
        bt_stride, positions, seq_idx, out, part_acc, part_ml, splits, Tn, H,
        C, R, bs, window, scale, sink, s);
}

#define LM_CASE(N, DEC, TH)                                                   \
    latent_attn_mfma_kernel<N, DEC><<<grid, TH, 0, s>>>(                      \
        (const unsigned short*)q_abs, (const unsigned short*)q_rot, qr_tok,   \
        qr_head, (const unsigned short*)gate, gate_tok,                       \
        (const unsigned short*)cache, block_table, bt_stride, cu, positions,  \
        seq_idx, (unsigned short*)out, part_acc, part_ml, Tn, H, C, R, bs,    \
        window, scale, sink)

// bf16 on the matrix cores: prompt portions (max_qlen >= 16; 16-query x
// 4-head workgroups over B sequences) or pure decode steps (max_qlen == 1;
// one wave per token x 16 heads x key split, merged by the combine kernel
// when splits > 1). Returns nonzero when the shape is not covered (latent
// or rotated width not a multiple of 8, or their sum above 576): the caller
// then uses the generic kernel.
extern "C" int launch_latent_attn_mfma(
    const void* q_abs, const void* q_rot, long qr_tok, long qr_head,
    const void* gate, long gate_tok, const void* cache,
    const int* block_table, int bt_stride, const int* cu,
    const int* positions, const int* seq_idx, void* out, float* part_acc,
    float* part_ml, int splits, int Tn, int B, int max_qlen, int H, int C,
    int R, int bs, int window, float scale, const float* sink,
    hipStream_t s) {
    const int Dk = C + R;
    if (C % 8 != 0 || R % 8 != 0 || Dk > 576) return 1;
    if (Tn == 0 || B == 0) return 0;
    const int ksteps = (Dk + 31) / 32;
    if (max_qlen == 1) {
        const dim3 grid(Tn, (H + 15) / 16, splits);
        if (ksteps <= 4) LM_CASE(4, true, 256);
        else if (ksteps <= 8) LM_CASE(8, true, 256);
        else if (ksteps <= 12) LM_CASE(12, true, 256);
        else LM_CASE(18, true, 256);
        if (splits > 1) {
            const dim3 g2(Tn, H);
            latent_attn_combine_kernel<unsigned short>
                <<<g2, LC_THREADS, 0, s>>>(
                    part_acc, part_ml, (const unsigned short*)gate, gate_tok,
                    (unsigned short*)out, splits, Tn, H, C, sink);
        }
        return 0;
    }
    const dim3 grid((max_qlen + 15) / 16, (H + 3) / 4, B);
    if (ksteps <= 4) LM_CASE(4, false, 256);
    else if (ksteps <= 8) LM_CASE(8, false, 256);
    else if (ksteps <= 12) LM_CASE(12, false, 256);
    else LM_CASE(18, false, 256);
    return 0;
}

#define LI_LAUNCH(N, MODE, GRID)                                              \
    lightning_kernel<TT, N, MODE, FORM>                                       \
        <<<GRID, LI_COLS * LI_GROUPS, 0, s>>>(                                \
            (const TT*)q, (const TT*)k, (const TT*)v, tok_stride, cos_t,      \
            sin_t, rdims, k_scale, decay, state, state_slots, cu, positions,  \
            out, ws, B, H, D, Dv)

#define LI_CASE(N)                                                            \
    case N:                                                                   \
        if (n_seg == 0) {                                                     \
            LI_LAUNCH(N, 0, grid);                                            \
        } else {                                                              \
            LI_LAUNCH(N, 1, sgrid);                                           \
            lightning_scan_kernel<<<scan_grid, 256, 0, s>>>(                  \
                decay, state, state_slots, cu, positions, ws, H, D * Dv);     \
            LI_LAUNCH(N, 2, sgrid);                                           \
        }                                                                     \
        break;

// n_seg = 0: one workgroup walks each whole chunk. n_seg > 0 (an upper bound
// of the number of LI_SEG-token segments in the batch, ws sized for it):
// segments run in parallel, a scan carries the state across them.
template <typename TT, int FORM>
static int lightning_dispatch(const void* q, const void* k, const void* v,
                              long tok_stride, const float* cos_t,
                              const float* sin_t, int rdims, float k_scale,
                              const float* decay,
                              float* state, const int* state_slots,
                              const int* cu, const int* positions, float* out,
                              float* ws, int n_seg, int B, int H, int D,
                              int Dv, hipStream_t s) {
    const int need = (D + LI_GROUPS - 1) / LI_GROUPS;
    const int sizes[] = {2, 8, 16, 32, 64};
    int dpt = 0;
    for (int z : sizes)
        if (z >= need) { dpt = z; break; }
    if (!dpt) return 1;
    const int zc = (Dv + LI_COLS - 1) / LI_COLS;
    const dim3 grid(B, H, zc), sgrid(n_seg > 0 ? n_seg : 1, H, zc);
    const dim3 scan_grid(B, H, (D * Dv + 255) / 256);
    switch (dpt) { LI_CASE(2) LI_CASE(8) LI_CASE(16) LI_CASE(32) LI_CASE(64) }
    return 0;
}

// returns nonzero when the key dim exceeds 256
extern "C" int lightning_segment_tokens() { return LI_SEG; }

// form 0: silu(q, k, v) (lightning); form 1: rotated q, k, scaled k, plain
// v (retention; cos_t/sin_t may be null when rdims is 0)
extern "C" int launch_lightning(const void* q, const void* k, const void* v,
                                long tok_stride, const float* decay,
                                float* state, const int* state_slots,
                                const int* cu, const int* positions,
                                float* out, float* ws, int n_seg, int B,
                                int H, int D, int Dv, int f32, int form,
                                const float* cos_t, const float* sin_t,
                                int rdims, float k_scale, hipStream_t s) {
    if (B == 0) return 0;
#define LI_DISPATCH(TT, FORM)                                                 \
    lightning_dispatch<TT, FORM>(q, k, v, tok_stride, cos_t, sin_t, rdims,    \
                                 k_scale, decay, state, state_slots, cu,      \
                                 positions, out, ws, n_seg, B, H, D, Dv, s)
    if (form == 0)
        return f32 ? LI_DISPATCH(float, 0) : LI_DISPATCH(unsigned short, 0);
    return f32 ? LI_DISPATCH(float, 1) : LI_DISPATCH(unsigned short, 1);
#undef LI_DISPATCH
}

#define DR_LAUNCH(N, R)                                                       \
    do {                                                                      \
        const dim3 grid(B, H, (Dv * R + WAVE - 1) / WAVE);                    \
        if (chdec)                                                            \
            delta_rule_kernel<N, R, true><<<grid, WAVE, 0, s>>>(              \
                q, k, qk_tok, v, v_tok, beta, g, state, state_slots, cu,      \
                positions, out, H, G, D, Dv);                                 \
        else                                                                  \
            delta_rule_kernel<N, R, false><<<grid, WAVE, 0, s>>>(             \
                q, k, qk_tok, v, v_tok, beta, g, state, state_slots, cu,      \
                positions, out, H, G, D, Dv);                                 \
    } while (0)

#define DR_CASE(N, R)                                                         \
    if (rg == R && dpt == N) { DR_LAUNCH(N, R); return 0; }

// returns nonzero when the key dim exceeds 256
extern "C" int launch_delta_rule(const float* q, const float* k, long qk_tok,
                                 const float* v, long v_tok,
                                 const float* beta, const float* g, int chdec,
                                 float* state, const int* state_slots,
                                 const int* cu, const int* positions,
                                 float* out, int B, int H, int G, int D,
                                 int Dv, hipStream_t s) {
    if (B == 0) return 0;
    if (D > 256) return 1;
    // row groups per column: 4 unless that leaves the chip short of about
    // four waves per SIMD (a few long portions), then 8 or 16
    int rg = 4;
    while (rg < 16 && (long)B * H * ((Dv * rg + WAVE - 1) / WAVE) < 4096)
        rg <<= 1;
    const int need = (D + rg - 1) / rg;
    const int dpt = need <= 4 ? 4 : need <= 8 ? 8 : need <= 16 ? 16
                    : need <= 32 ? 32 : 64;
    DR_CASE(4, 4) DR_CASE(8, 4) DR_CASE(16, 4) DR_CASE(32, 4) DR_CASE(64, 4)
    DR_CASE(4, 8) DR_CASE(8, 8) DR_CASE(16, 8) DR_CASE(32, 8)
    DR_CASE(4, 16) DR_CASE(8, 16) DR_CASE(16, 16)
    return 1;
}

#define SA_LAUNCH(N, R, P)                                                    \
    sink_attn_kernel<TT, N, R, P><<<grid, SA_WAVES * WAVE, smem, s>>>(        \
        (const TT*)q, q_tok, (const TT*)k_cache, (const TT*)v_cache,          \
        block_table, bt_stride, positions, seq_idx, sink, (TT*)out, out_tok,  \
        out_scale, part_acc, part_ml, Tn, H, G, D, Dv, bs, window,            \
        (const TT*)head_gate, hg_tok)

#define SA_CASE(N, P)                                                         \
    if (dpl == N && pair == P) {                                              \
        if (rep == 4) SA_LAUNCH(N, 4, P);                                     \
        else if (rep == 2) SA_LAUNCH(N, 2, P);                                \
        else SA_LAUNCH(N, 1, P);                                              \
        launched = true;                                                      \
    }

template <typename TT>
static int sink_attn_dispatch(const void* q, long q_tok, const void* k_cache,
                              const void* v_cache, const int* block_table,
                              int bt_stride, const int* positions,
                              const int* seq_idx, const float* sink,
                              void* out, long out_tok, float out_scale,
                              float* part_acc, float* part_ml, int splits,
                              int Tn, int H, int G, int D, int Dv, int bs,
                              int window, const void* head_gate, long hg_tok,
                              hipStream_t s) {
    // even value sizes: a lane owns coordinate pairs (one load for two)
    const bool pair = Dv % 2 == 0;
    int dpl = pair ? 2 * ((Dv + 2 * WAVE - 1) / (2 * WAVE))
                   : (Dv + WAVE - 1) / WAVE;
    if (dpl == 3) dpl = 4;
    // query heads per wave: the largest of 4, 2, 1 that divides the group
    const int group = H / G;
    const int rep = group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1;
    const int units = H / rep;
    const size_t smem = (size_t)SA_WAVES * rep * D * sizeof(float);
    const dim3 grid(Tn, (units + SA_WAVES - 1) / SA_WAVES, splits);
    bool launched = false;
    SA_CASE(2, true) SA_CASE(4, true)
    SA_CASE(1, false) SA_CASE(2, false) SA_CASE(4, false)
    if (!launched) return 1;
    if (splits > 1) {
        const dim3 g2(Tn, (H + SA_WAVES - 1) / SA_WAVES);
        sink_attn_combine_kernel<TT><<<g2, SA_WAVES * WAVE, 0, s>>>(
            part_acc, part_ml, sink, (TT*)out, out_tok, out_scale, splits, Tn,
            H, Dv, (const TT*)head_gate, hg_tok);
    }
    return 0;
}

// head_gate (optional, activation type, [Tn, H] with row stride hg_tok):
// head h's output times sigmoid(head_gate[t, h]). Returns nonzero when a
// head size exceeds 256.
extern "C" int launch_sink_attn(const void* q, long q_tok,
                                const void* k_cache, const void* v_cache,
                                const int* block_table, int bt_stride,
                                const int* positions, const int* seq_idx,
                                const float* sink, void* out, long out_tok,
                                float out_scale, float* part_acc,
                                float* part_ml, int splits, int Tn, int H,
                                int G, int D, int Dv, int bs, int window,
                                int f32, const void* head_gate, long hg_tok,
                                hipStream_t s) {
    if (D > SA_MAXD || Dv > SA_MAXD) return 1;
    if (Tn == 0) return 0;
    if (f32)
        return sink_attn_dispatch<float>(
            q, q_tok, k_cache, v_cache, block_table, bt_stride, positions,
            seq_idx, sink, out, out_tok, out_scale, part_acc, part_ml, splits,
            Tn, H, G, D, Dv, bs, window, head_gate, hg_tok, s);
    return sink_attn_dispatch<unsigned short>(
        q, q_tok, k_cache, v_cache, block_table, bt_stride, positions,
        seq_idx, sink, out, out_tok, out_scale, part_acc, part_ml, splits, Tn,
        H, G, D, Dv, bs, window, head_gate, hg_tok, s);
}

// ---------------------------------------------------------------------------
// talk_attn: windowed grouped-query softmax attention whose per-head softmax
// weights are mixed across heads before they meet the values,
//   w'_h = sum_g talk[h, g] w_g,   o_h = sum_j w'_h(j) v_{c(h)}(j),
// c(h) the key/value head of query head h. Since the mix is linear,
//   o_h = sum_g talk[h, g] A[g, c(h)],   A[g, c] = sum_j w_g(j) v_c(j):
// every query head's ordinary softmax weights are applied to the values of
// EVERY key/value head (kernel 1, online softmax, key-split capable), and a
// second kernel merges the key splits, normalizes, mixes the heads with
// `talk`, applies the sigmoid output gate and writes the activation.
//
// Kernel 1 keeps sink_attn's wave layout: one wave per (token, REP query
// heads of one key group, block of NV value heads, key split); lane = key
// for the scores, lane = coordinate pair for the value sums. Partials:
// part_acc [S, T, G, H, Dv] (unnormalized), part_ml [S, T, H, 2].
namespace {

template <typename T, int DPL, int REP, int NV, bool PAIR>
__global__ void __launch_bounds__(SA_WAVES * WAVE)
talk_attn_kernel(const T* __restrict__ q, long q_tok,
                 const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                 const int* __restrict__ block_table, int bt_stride,
                 const int* __restrict__ positions,
                 const int* __restrict__ seq_idx,
                 float* __restrict__ part_acc, float* __restrict__ part_ml,
                 int Tn, int H, int G, int D, int Dv, int bs, int window,
                 int units, int vblocks) {
    extern __shared__ __attribute__((aligned(16))) float sa_q[];
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int t = blockIdx.x;
    const int u = blockIdx.y * SA_WAVES + wid;
    if (u >= units * vblocks) return;      // no workgroup barrier below
    const int h0 = (u % units) * REP;      // REP consecutive query heads
    const int v0 = (u / units) * NV;       // NV consecutive value heads
    const int split = blockIdx.z, nsplit = gridDim.z;
    const int p = positions[t];
    const int g = h0 / (H / G);
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int per =
        ((p + 1 - lo + nsplit - 1) / nsplit + WAVE - 1) / WAVE * WAVE;
    const int klo = lo + split * per, khi = min(p + 1, klo + per);
    float* qv = sa_q + (long)wid * REP * D;
    for (int i = lane; i < REP * D; i += WAVE)
        qv[i] = ldf(q + (long)t * q_tok + (long)h0 * D + i);
    WAVE_LDS_SYNC();
    const int* bt = block_table + (long)seq_idx[t] * bt_stride;
    float m[REP], l[REP], acc[NV][REP][DPL];
#pragma unroll
    for (int r = 0; r < REP; ++r) {
        m[r] = -INFINITY;
        l[r] = 0.f;
#pragma unroll
        for (int n = 0; n < NV; ++n)
#pragma unroll
            for (int i = 0; i < DPL; ++i) acc[n][r][i] = 0.f;
    }
    for (int j0 = klo; j0 < khi; j0 += WAVE) {
        const int j = j0 + lane;
        const bool valid = j < khi;
        int row0 = 0;           // row of key head 0; lanes past the end
        float sc[REP], pj[REP]; // point at a real row
#pragma unroll
        for (int r = 0; r < REP; ++r) sc[r] = 0.f;
        const int nk = min(WAVE, khi - j0);
        {   // past the end: the share's last key, a row the sequence wrote
            const int jc = min(j, khi - 1);
            row0 = bt[jc / bs] * G * bs + jc % bs;
        }
        if (valid)
            SaDots<T, REP>::run(k_cache + (long)(row0 + g * bs) * D, qv, D,
                                sc);
#pragma unroll
        for (int r = 0; r < REP; ++r) {
            const float s = valid ? sc[r] : -INFINITY;
            const float m_new = fmaxf(m[r], wave_max(s));
            pj[r] = valid ? expf(s - m_new) : 0.f;
            const float corr = expf(m[r] - m_new);
            l[r] = l[r] * corr + wave_sum(pj[r]);
#pragma unroll
            for (int n = 0; n < NV; ++n)
#pragma unroll
                for (int i = 0; i < DPL; ++i) acc[n][r][i] *= corr;
            m[r] = m_new;
        }
#pragma unroll
        for (int n = 0; n < NV; ++n) {
            if (v0 + n >= G) break;
            for (int jj = 0; jj < nk; jj += SA_PV) {
                float vv[SA_PV][DPL];
#pragma unroll
                for (int x = 0; x < SA_PV; ++x) {
                    const T* vr =
                        v_cache +
                        (long)(__builtin_amdgcn_readlane(row0, jj + x) +
                               (v0 + n) * bs) * Dv;
                    if constexpr (PAIR) {
#pragma unroll
                        for (int i = 0; i < DPL; i += 2) {
                            const int d = sa_coord<true>(lane, i);
                            vv[x][i] = vv[x][i + 1] = 0.f;
                            if (d < Dv) sa_ld2(vr + d, vv[x][i], vv[x][i + 1]);
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < DPL; ++i) {
                            const int d = sa_coord<false>(lane, i);
                            vv[x][i] = d < Dv ? ldf(vr + d) : 0.f;
                        }
                    }
                }
#pragma unroll
                for (int x = 0; x < SA_PV; ++x)
#pragma unroll
                    for (int r = 0; r < REP; ++r) {
                        const float pb = __builtin_bit_cast(
                            float, __builtin_amdgcn_readlane(
                                       __builtin_bit_cast(int, pj[r]), jj + x));
#pragma unroll
                        for (int i = 0; i < DPL; ++i)
                            acc[n][r][i] += pb * vv[x][i];
                    }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < REP; ++r) {
        const int h = h0 + r;
        const long prow = ((long)split * Tn + t) * H + h;
        if (lane == 0 && v0 == 0) {
            part_ml[prow * 2] = m[r];
            part_ml[prow * 2 + 1] = l[r];
        }
#pragma unroll
        for (int n = 0; n < NV; ++n) {
            if (v0 + n >= G) break;
#pragma unroll
            for (int i = 0; i < DPL; ++i) {
                const int d = sa_coord<PAIR>(lane, i);
                if (d < Dv)
                    part_acc[((((long)split * Tn + t) * G + v0 + n) * H + h) *
                                 Dv + d] = acc[n][r][i];
            }
        }
    }
}

// Merge of the key splits + head mix + output gate. Workgroup per (token,
// key/value head c): the merged, normalized sums A[g, c] of all query heads
// g are staged in LDS, then every query head of group c takes its mixture.
// part_ml == nullptr: the partials are already normalized (one split).
// LDS: wts [S*H] | talk rows of the group [rep*H] | A_c [H*Dv].
template <typename T>
__global__ void __launch_bounds__(256)
talk_mix_kernel(const float* __restrict__ part_acc,
                const float* __restrict__ part_ml,
                const float* __restrict__ talk, const T* __restrict__ gate,
                long gate_tok, T* __restrict__ out, long out_tok, int splits,
                int Tn, int H, int G, int Dv) {
    extern __shared__ __attribute__((aligned(16))) float tm_s[];
    const int rep = H / G;
    float* wts = tm_s;
    float* tk = wts + splits * H;
    float* A = tk + rep * H;
    const int t = blockIdx.x, c = blockIdx.y;
    for (int h = threadIdx.x; h < H; h += blockDim.x) {
        if (!part_ml) {
            wts[h] = 1.f;
            continue;
        }
        float M = -INFINITY;
        for (int s = 0; s < splits; ++s) {
            const long row = ((long)s * Tn + t) * H + h;
            if (part_ml[row * 2 + 1] > 0.f) M = fmaxf(M, part_ml[row * 2]);
        }
        float L = 0.f;
        for (int s = 0; s < splits; ++s) {
            const long row = ((long)s * Tn + t) * H + h;
            const float l = part_ml[row * 2 + 1];
            const float w = l > 0.f ? expf(part_ml[row * 2] - M) : 0.f;
            wts[s * H + h] = w;
            L += l * w;
        }
        const float rcp = L > 0.f ? 1.f / L : 0.f;
        for (int s = 0; s < splits; ++s) wts[s * H + h] *= rcp;
    }
    for (int i = threadIdx.x; i < rep * H; i += blockDim.x)
        tk[i] = talk[(long)c * rep * H + i];
    __syncthreads();
    for (int idx = threadIdx.x; idx < H * Dv; idx += blockDim.x) {
        const int gq = idx / Dv, d = idx - gq * Dv;
        float a = 0.f;
        for (int s = 0; s < splits; ++s)
            a += wts[s * H + gq] *
                 part_acc[((((long)s * Tn + t) * G + c) * H + gq) * Dv + d];
        A[idx] = a;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < rep * Dv; idx += blockDim.x) {
        const int hl = idx / Dv, d = idx - hl * Dv;
        const int h = c * rep + hl;
        float o = 0.f;
        for (int gq = 0; gq < H; ++gq) o += tk[hl * H + gq] * A[gq * Dv + d];
        const float gt = ldf(gate + (long)t * gate_tok + (long)h * Dv + d);
        stf(out + (long)t * out_tok + (long)h * Dv + d, o / (1.f + expf(-gt)));
    }
}

}  // namespace

// ---------------------------------------------------------------------------
// The same attention for steps whose score matrix is small (decode rows,
// short portions, windows): the raw scores of every (token, head, visible
// key) are written once (kernel 1, with the per-split max/sum), and kernel
// 2 turns them into normalized weights of ALL heads, mixes them with the
// wave's rows of `talk` — w'_h(j) = sum_g talk[h, g] w_g(j) — and applies
// the mixed weights to the values of the wave's own key/value head only:
// each cached value row is read once per key group, as in plain attention.
// scores [Tn, H, ctx] fp32, entry (j - lo) of a row whose first visible
// key is lo. Wave layout as above: (token, REP query heads of one key
// group, key split); lane = key for scores and weights, lane = coordinate
// pair for the value sum.
namespace {

template <typename T, int REP>
__global__ void __launch_bounds__(SA_WAVES * WAVE)
talk_scores_kernel(const T* __restrict__ q, long q_tok,
                   const T* __restrict__ k_cache,
                   const int* __restrict__ block_table, int bt_stride,
                   const int* __restrict__ positions,
                   const int* __restrict__ seq_idx,
                   float* __restrict__ scores, long ctx,
                   float* __restrict__ part_ml, int Tn, int H, int G, int D,
                   int bs, int window, float softcap) {
    extern __shared__ __attribute__((aligned(16))) float sa_q[];
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int t = blockIdx.x;
    const int unit = blockIdx.y * SA_WAVES + wid;
    if (unit * REP >= H) return;      // no workgroup barrier below
    const int h0 = unit * REP;
    const int split = blockIdx.z, nsplit = gridDim.z;
    const int p = positions[t];
    const int g = h0 / (H / G);
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int per =
        ((p + 1 - lo + nsplit - 1) / nsplit + WAVE - 1) / WAVE * WAVE;
    const int klo = lo + split * per, khi = min(p + 1, klo + per);
    float* qv = sa_q + (long)wid * REP * D;
    for (int i = lane; i < REP * D; i += WAVE)
        qv[i] = ldf(q + (long)t * q_tok + (long)h0 * D + i);
    WAVE_LDS_SYNC();
    const int* bt = block_table + (long)seq_idx[t] * bt_stride;
    float m[REP], l[REP];
#pragma unroll
    for (int r = 0; r < REP; ++r) {
        m[r] = -INFINITY;
        l[r] = 0.f;
    }
    for (int j0 = klo; j0 < khi; j0 += WAVE) {
        const int j = j0 + lane;
        const bool valid = j < khi;
        float sc[REP];
#pragma unroll
        for (int r = 0; r < REP; ++r) sc[r] = 0.f;
        if (valid) {
            const int row = (bt[j / bs] * G + g) * bs + j % bs;
            SaDots<T, REP>::run(k_cache + (long)row * D, qv, D, sc);
        }
#pragma unroll
        for (int r = 0; r < REP; ++r) {
            // softcap > 0: the stored score is softcap * tanh(s / softcap)
            if (softcap > 0.f) sc[r] = softcap * tanhf(sc[r] / softcap);
            const float sv = valid ? sc[r] : -INFINITY;
            if (valid)
                scores[((long)t * H + h0 + r) * ctx + (j - lo)] = sv;
            const float m_new = fmaxf(m[r], wave_max(sv));
            const float e = valid ? expf(sv - m_new) : 0.f;
            l[r] = l[r] * expf(m[r] - m_new) + wave_sum(e);
            m[r] = m_new;
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < REP; ++r) {
            const long prow = ((long)split * Tn + t) * H + h0 + r;
            part_ml[prow * 2] = m[r];
            part_ml[prow * 2 + 1] = l[r];
        }
    }
}

// ml_splits: the number of key splits kernel 1 ran with (rows of part_ml).
// Per-wave LDS: max [H] | 1/sum [H] | talk rows [REP*H].
template <typename T, int DPL, int REP, bool PAIR>
__global__ void __launch_bounds__(SA_WAVES * WAVE)
talk_pv_kernel(const float* __restrict__ scores, long ctx,
               const float* __restrict__ part_ml, int ml_splits,
               const float* __restrict__ talk,
               const T* __restrict__ v_cache,
               const int* __restrict__ block_table, int bt_stride,
               const int* __restrict__ positions,
               const int* __restrict__ seq_idx, const T* __restrict__ gate,
               long gate_tok, T* __restrict__ out, long out_tok,
               float* __restrict__ part_o, int Tn, int H, int G, int Dv,
               int bs, int window) {
    extern __shared__ __attribute__((aligned(16))) float tp_s[];
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int t = blockIdx.x;
    const int unit = blockIdx.y * SA_WAVES + wid;
    if (unit * REP >= H) return;      // no workgroup barrier below
    const int h0 = unit * REP;
    const int split = blockIdx.z, nsplit = gridDim.z;
    const int p = positions[t];
    const int g = h0 / (H / G);
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int per =
        ((p + 1 - lo + nsplit - 1) / nsplit + WAVE - 1) / WAVE * WAVE;
    const int klo = lo + split * per, khi = min(p + 1, klo + per);
    float* Mh = tp_s + (long)wid * (2 + REP) * H;
    float* iL = Mh + H;
    float* tkw = iL + H;
    for (int h = lane; h < H; h += WAVE) {
        float M = -INFINITY;
        for (int s = 0; s < ml_splits; ++s) {
            const long row = ((long)s * Tn + t) * H + h;
            if (part_ml[row * 2 + 1] > 0.f) M = fmaxf(M, part_ml[row * 2]);
        }
        float L = 0.f;
        for (int s = 0; s < ml_splits; ++s) {
            const long row = ((long)s * Tn + t) * H + h;
            const float l = part_ml[row * 2 + 1];
            if (l > 0.f) L += l * expf(part_ml[row * 2] - M);
        }
        Mh[h] = M;
        iL[h] = L > 0.f ? 1.f / L : 0.f;
    }
    for (int i = lane; i < REP * H; i += WAVE)
        tkw[i] = talk[(long)h0 * H + i];
    WAVE_LDS_SYNC();
    const int* bt = block_table + (long)seq_idx[t] * bt_stride;
    float acc[REP][DPL];
#pragma unroll
    for (int r = 0; r < REP; ++r)
#pragma unroll
        for (int i = 0; i < DPL; ++i) acc[r][i] = 0.f;
    const float* srow = scores + (long)t * H * ctx;
    for (int j0 = klo; j0 < khi; j0 += WAVE) {
        const int j = j0 + lane;
        const bool valid = j < khi;
        const int nk = min(WAVE, khi - j0);
        // lanes past the end point at the share's last key: a row this
        // sequence wrote (their weights are 0, and 0 x garbage is not 0)
        const int jc = min(j, khi - 1);
        const int row = (bt[jc / bs] * G + g) * bs + jc % bs;
        float pj[REP];
#pragma unroll
        for (int r = 0; r < REP; ++r) pj[r] = 0.f;
        if (valid) {
            for (int gq = 0; gq < H; ++gq) {
                const float e =
                    expf(srow[(long)gq * ctx + (j - lo)] - Mh[gq]) * iL[gq];
#pragma unroll
                for (int r = 0; r < REP; ++r) pj[r] += tkw[r * H + gq] * e;
            }
        }
#pragma unroll 2
        for (int jj = 0; jj < nk; jj += SA_PV) {
            float vv[SA_PV][DPL];
#pragma unroll
            for (int x = 0; x < SA_PV; ++x) {
                const T* vr =
                    v_cache + (long)__builtin_amdgcn_readlane(row, jj + x) * Dv;
                if constexpr (PAIR) {
#pragma unroll
                    for (int i = 0; i < DPL; i += 2) {
                        const int d = sa_coord<true>(lane, i);
                        vv[x][i] = vv[x][i + 1] = 0.f;
                        if (d < Dv) sa_ld2(vr + d, vv[x][i], vv[x][i + 1]);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < DPL; ++i) {
                        const int d = sa_coord<false>(lane, i);
                        vv[x][i] = d < Dv ? ldf(vr + d) : 0.f;
                    }
                }
            }
#pragma unroll
            for (int x = 0; x < SA_PV; ++x)
#pragma unroll
                for (int r = 0; r < REP; ++r) {
                    const float pb = __builtin_bit_cast(
                        float, __builtin_amdgcn_readlane(
                                   __builtin_bit_cast(int, pj[r]), jj + x));
#pragma unroll
                    for (int i = 0; i < DPL; ++i) acc[r][i] += pb * vv[x][i];
                }
        }
    }
#pragma unroll
    for (int r = 0; r < REP; ++r) {
        const int h = h0 + r;
#pragma unroll
        for (int i = 0; i < DPL; ++i) {
            const int d = sa_coord<PAIR>(lane, i);
            if (d >= Dv) continue;
            if (nsplit == 1) {
                const float gt =
                    ldf(gate + (long)t * gate_tok + (long)h * Dv + d);
                stf(out + (long)t * out_tok + (long)h * Dv + d,
                    acc[r][i] / (1.f + expf(-gt)));
            } else {
                part_o[(((long)split * Tn + t) * H + h) * Dv + d] = acc[r][i];
            }
        }
    }
}

// out = sigmoid(gate) * sum over splits of part_o [S, Tn, H*Dv]
template <typename T>
__global__ void talk_sum_gate_kernel(const float* __restrict__ part_o,
                                     const T* __restrict__ gate, long gate_tok,
                                     T* __restrict__ out, long out_tok,
                                     int splits, int Tn, int N) {
    const int t = blockIdx.x;
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < N;
         i += gridDim.y * blockDim.x) {
        float a = 0.f;
        for (int s = 0; s < splits; ++s)
            a += part_o[((long)s * Tn + t) * N + i];
        const float gt = ldf(gate + (long)t * gate_tok + i);
        stf(out + (long)t * out_tok + i, a / (1.f + expf(-gt)));
    }
}

}  // namespace

#define TP_LAUNCH(N, R, P)                                                    \
    talk_pv_kernel<TT, N, R, P><<<grid, SA_WAVES * WAVE, smem2, s>>>(         \
        scores, ctx, part_ml, splits, talk, (const TT*)v_cache, block_table,  \
        bt_stride, positions, seq_idx, (const TT*)gate, gate_tok, (TT*)out,   \
        out_tok, part_o, Tn, H, G, Dv, bs, window)

#define TP_CASE(N, P)                                                         \
    if (dpl == N && pair == P) {                                              \
        if (rep == 4) TP_LAUNCH(N, 4, P);                                     \
        else if (rep == 2) TP_LAUNCH(N, 2, P);                                \
        else TP_LAUNCH(N, 1, P);                                              \
        launched = true;                                                      \
    }

template <typename TT>
static int talk_scored_dispatch(const void* q, long q_tok, const void* k_cache,
                                const void* v_cache, const int* block_table,
                                int bt_stride, const int* positions,
                                const int* seq_idx, const float* talk,
                                const void* gate, long gate_tok, void* out,
                                long out_tok, float* scores, long ctx,
                                float* part_ml, float* part_o, int splits,
                                int Tn, int H, int G, int D, int Dv, int bs,
                                int window, hipStream_t s) {
    const bool pair = Dv % 2 == 0;
    int dpl = pair ? 2 * ((Dv + 2 * WAVE - 1) / (2 * WAVE))
                   : (Dv + WAVE - 1) / WAVE;
    if (dpl == 3) dpl = 4;
    const int group = H / G;
    const int rep = group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1;
    const int units = H / rep;
    const dim3 grid(Tn, (units + SA_WAVES - 1) / SA_WAVES, splits);
    const size_t smem1 = (size_t)SA_WAVES * rep * D * sizeof(float);
    const size_t smem2 = (size_t)SA_WAVES * (2 + rep) * H * sizeof(float);
#define TS_LAUNCH(R)                                                          \
    talk_scores_kernel<TT, R><<<grid, SA_WAVES * WAVE, smem1, s>>>(           \
        (const TT*)q, q_tok, (const TT*)k_cache, block_table, bt_stride,      \
        positions, seq_idx, scores, ctx, part_ml, Tn, H, G, D, bs, window,    \
        0.f)
    if (rep == 4) TS_LAUNCH(4);
    else if (rep == 2) TS_LAUNCH(2);
    else TS_LAUNCH(1);
#undef TS_LAUNCH
    bool launched = false;
    TP_CASE(2, true) TP_CASE(4, true)
    TP_CASE(1, false) TP_CASE(2, false) TP_CASE(4, false)
    if (!launched) return 1;
    if (splits > 1) {
        const int N = H * Dv;
        const dim3 g2(Tn, (N + 255) / 256);
        talk_sum_gate_kernel<TT><<<g2, 256, 0, s>>>(
            part_o, (const TT*)gate, gate_tok, (TT*)out, out_tok, splits, Tn,
            N);
    }
    return 0;
}

// Scores written once, then mixed weights against each head's own values.
// scores [Tn, H, ctx], part_ml [splits, Tn, H, 2], part_o [splits, Tn, H,
// Dv] (unused when splits == 1); nonzero when a head size exceeds 256.
extern "C" int launch_talk_attn_scored(
    const void* q, long q_tok, const void* k_cache, const void* v_cache,
    const int* block_table, int bt_stride, const int* positions,
    const int* seq_idx, const float* talk, const void* gate, long gate_tok,
    void* out, long out_tok, float* scores, long ctx, float* part_ml,
    float* part_o, int splits, int Tn, int H, int G, int D, int Dv, int bs,
    int window, int f32, hipStream_t s) {
    if (D > SA_MAXD || Dv > SA_MAXD) return 1;
    if (Tn == 0) return 0;
    if (f32)
        return talk_scored_dispatch<float>(
            q, q_tok, k_cache, v_cache, block_table, bt_stride, positions,
            seq_idx, talk, gate, gate_tok, out, out_tok, scores, ctx, part_ml,
            part_o, splits, Tn, H, G, D, Dv, bs, window, s);
    return talk_scored_dispatch<unsigned short>(
        q, q_tok, k_cache, v_cache, block_table, bt_stride, positions,
        seq_idx, talk, gate, gate_tok, out, out_tok, scores, ctx, part_ml,
        part_o, splits, Tn, H, G, D, Dv, bs, window, s);
}

#define TA_LAUNCH(N, R, V, P)                                                 \
    talk_attn_kernel<TT, N, R, V, P><<<grid, SA_WAVES * WAVE, smem, s>>>(     \
        (const TT*)q, q_tok, (const TT*)k_cache, (const TT*)v_cache,          \
        block_table, bt_stride, positions, seq_idx, part_acc, part_ml, Tn, H, \
        G, D, Dv, bs, window, units, vblocks)

#define TA_CASE(N, P)                                                         \
    if (dpl == N && pair == P) {                                              \
        if (rep == 4 && nv == 4) TA_LAUNCH(N, 4, 4, P);                       \
        else if (rep == 4 && nv == 2) TA_LAUNCH(N, 4, 2, P);                  \
        else if (rep == 4) TA_LAUNCH(N, 4, 1, P);                             \
        else if (rep == 2 && nv == 4) TA_LAUNCH(N, 2, 4, P);                  \
        else if (rep == 2 && nv == 2) TA_LAUNCH(N, 2, 2, P);                  \
        else if (rep == 2) TA_LAUNCH(N, 2, 1, P);                             \
        else if (nv == 4) TA_LAUNCH(N, 1, 4, P);                              \
        else if (nv == 2) TA_LAUNCH(N, 1, 2, P);                              \
        else TA_LAUNCH(N, 1, 1, P);                                           \
        launched = true;                                                      \
    }

template <typename TT>
static int talk_attn_dispatch(const void* q, long q_tok, const void* k_cache,
                              const void* v_cache, const int* block_table,
                              int bt_stride, const int* positions,
                              const int* seq_idx, float* part_acc,
                              float* part_ml, int splits, int Tn, int H,
                              int G, int D, int Dv, int bs, int window,
                              hipStream_t s) {
    const bool pair = Dv % 2 == 0;
    int dpl = pair ? 2 * ((Dv + 2 * WAVE - 1) / (2 * WAVE))
                   : (Dv + WAVE - 1) / WAVE;
    if (dpl == 3) dpl = 4;
    const int group = H / G;
    const int rep = group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1;
    // value heads per wave: scores are recomputed per block of value heads
    const int nv = G >= 4 ? 4 : G >= 2 ? 2 : 1;
    const int units = H / rep;
    const int vblocks = (G + nv - 1) / nv;
    const size_t smem = (size_t)SA_WAVES * rep * D * sizeof(float);
    const dim3 grid(Tn, (units * vblocks + SA_WAVES - 1) / SA_WAVES, splits);
    bool launched = false;
    TA_CASE(2, true) TA_CASE(4, true)
    TA_CASE(1, false) TA_CASE(2, false) TA_CASE(4, false)
    return launched ? 0 : 1;
}

// Scores and per-value-head sums into the partial buffers; nonzero when a
// head size exceeds 256.
extern "C" int launch_talk_attn(const void* q, long q_tok,
                                const void* k_cache, const void* v_cache,
                                const int* block_table, int bt_stride,
                                const int* positions, const int* seq_idx,
                                float* part_acc, float* part_ml, int splits,
                                int Tn, int H, int G, int D, int Dv, int bs,
                                int window, int f32, hipStream_t s) {
    if (D > SA_MAXD || Dv > SA_MAXD) return 1;
    if (Tn == 0) return 0;
    if (f32)
        return talk_attn_dispatch<float>(
            q, q_tok, k_cache, v_cache, block_table, bt_stride, positions,
            seq_idx, part_acc, part_ml, splits, Tn, H, G, D, Dv, bs, window,
            s);
    return talk_attn_dispatch<unsigned short>(
        q, q_tok, k_cache, v_cache, block_table, bt_stride, positions,
        seq_idx, part_acc, part_ml, splits, Tn, H, G, D, Dv, bs, window, s);
}

// Split merge + head mix + sigmoid gate -> out; nonzero when the LDS need
// exceeds 64 KB.
extern "C" int launch_talk_mix(const float* part_acc, const float* part_ml,
                               const float* talk, const void* gate,
                               long gate_tok, void* out, long out_tok,
                               int splits, int Tn, int H, int G, int Dv,
                               int f32, hipStream_t s) {
    if (Tn == 0) return 0;
    const size_t smem = ((size_t)splits * H + (size_t)(H / G) * H +
                         (size_t)H * Dv) * sizeof(float);
    if (smem > 64 * 1024) return 1;
    const dim3 grid(Tn, G);
    if (f32)
        talk_mix_kernel<float><<<grid, 256, smem, s>>>(
            part_acc, part_ml, talk, (const float*)gate, gate_tok,
            (float*)out, out_tok, splits, Tn, H, G, Dv);
    else
        talk_mix_kernel<unsigned short><<<grid, 256, smem, s>>>(
            part_acc, part_ml, talk, (const unsigned short*)gate, gate_tok,
            (unsigned short*)out, out_tok, splits, Tn, H, G, Dv);
    return 0;
}


// ---------------------------------------------------------------------------
// mixed_score_attn: windowed grouped-query softmax attention whose (capped)
// scores are mixed across heads BEFORE the softmax,
//   s'_h(j) = sum_g mix[h, g] s_g(j),   o_h = softmax_j(s'_h) v_{c(h)}(j),
// c(h) the key/value head of query head h. Kernel 1 (talk_scores_kernel
// with its cap) writes every head's score of every visible key once; kernel
// 2 below reads, per key, the scores of ALL heads, mixes them with the
// wave's rows of `mix`, and runs sink_attn's online softmax and value sum on
// the mixed scores: wave = (token, REP query heads of one key group, key
// split), lane = key for the scores, lane = coordinate pair for the value
// sum, each cached value row read once per key group. Partials and the merge
// are sink_attn's (sink_attn_combine_kernel), so an optional sink logit and
// a per-head sigmoid gate come with it.
namespace {

template <typename T, int DPL, int REP, bool PAIR>
__global__ void __launch_bounds__(SA_WAVES * WAVE)
mixed_score_pv_kernel(const float* __restrict__ scores, long ctx,
                      const float* __restrict__ mix,
                      const T* __restrict__ v_cache,
                      const int* __restrict__ block_table, int bt_stride,
                      const int* __restrict__ positions,
                      const int* __restrict__ seq_idx,
                      const float* __restrict__ sink, T* __restrict__ out,
                      long out_tok, float* __restrict__ part_acc,
                      float* __restrict__ part_ml, int Tn, int H, int G,
                      int Dv, int bs, int window,
                      const T* __restrict__ head_gate, long hg_tok) {
    extern __shared__ __attribute__((aligned(16))) float ms_s[];
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int t = blockIdx.x;
    const int unit = blockIdx.y * SA_WAVES + wid;
    if (unit * REP >= H) return;      // no workgroup barrier below
    const int h0 = unit * REP;
    const int split = blockIdx.z, nsplit = gridDim.z;
    const int p = positions[t];
    const int g = h0 / (H / G);
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int per =
        ((p + 1 - lo + nsplit - 1) / nsplit + WAVE - 1) / WAVE * WAVE;
    const int klo = lo + split * per, khi = min(p + 1, klo + per);
    float* mw = ms_s + (long)wid * REP * H;         // the wave's rows of mix
    for (int i = lane; i < REP * H; i += WAVE) mw[i] = mix[(long)h0 * H + i];
    WAVE_LDS_SYNC();
    const int* bt = block_table + (long)seq_idx[t] * bt_stride;
    const float* srow = scores + (long)t * H * ctx;
    float m[REP], l[REP], acc[REP][DPL];
#pragma unroll
    for (int r = 0; r < REP; ++r) {
        m[r] = -INFINITY;
        l[r] = 0.f;
#pragma unroll
        for (int i = 0; i < DPL; ++i) acc[r][i] = 0.f;
    }
    for (int j0 = klo; j0 < khi; j0 += WAVE) {
        const int j = j0 + lane;
        const bool valid = j < khi;
        const int nk = min(WAVE, khi - j0);
        // lanes past the end point at the share's last key: a row this
        // sequence wrote (their weights are 0, and 0 x garbage is not 0)
        const int jc = min(j, khi - 1);
        const int row = (bt[jc / bs] * G + g) * bs + jc % bs;
        float sc[REP], pj[REP];
#pragma unroll
        for (int r = 0; r < REP; ++r) sc[r] = 0.f;
        if (valid) {
            for (int gq = 0; gq < H; ++gq) {
                const float sv = srow[(long)gq * ctx + (j - lo)];
#pragma unroll
                for (int r = 0; r < REP; ++r) sc[r] += mw[r * H + gq] * sv;
            }
        }
#pragma unroll
        for (int r = 0; r < REP; ++r) {
            const float sv = valid ? sc[r] : -INFINITY;
            const float m_new = fmaxf(m[r], wave_max(sv));
            pj[r] = valid ? expf(sv - m_new) : 0.f;
            const float corr = expf(m[r] - m_new);
            l[r] = l[r] * corr + wave_sum(pj[r]);
#pragma unroll
            for (int i = 0; i < DPL; ++i) acc[r][i] *= corr;
            m[r] = m_new;
        }
#pragma unroll 2
        for (int jj = 0; jj < nk; jj += SA_PV) {
            float vv[SA_PV][DPL];
#pragma unroll
            for (int u = 0; u < SA_PV; ++u) {
                const T* vr =
                    v_cache + (long)__builtin_amdgcn_readlane(row, jj + u) * Dv;
                if constexpr (PAIR) {
#pragma unroll
                    for (int i = 0; i < DPL; i += 2) {
                        const int d = sa_coord<true>(lane, i);
                        vv[u][i] = vv[u][i + 1] = 0.f;
                        if (d < Dv) sa_ld2(vr + d, vv[u][i], vv[u][i + 1]);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < DPL; ++i) {
                        const int d = sa_coord<false>(lane, i);
                        vv[u][i] = d < Dv ? ldf(vr + d) : 0.f;
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < SA_PV; ++u)
#pragma unroll
                for (int r = 0; r < REP; ++r) {
                    const float pb = __builtin_bit_cast(
                        float, __builtin_amdgcn_readlane(
                                   __builtin_bit_cast(int, pj[r]), jj + u));
#pragma unroll
                    for (int i = 0; i < DPL; ++i) acc[r][i] += pb * vv[u][i];
                }
        }
    }
#pragma unroll
    for (int r = 0; r < REP; ++r) {
        const int h = h0 + r;
        if (nsplit == 1) {
            float L = l[r], w = 1.f;
            if (sink) {
                const float sk = sink[h];
                const float M = fmaxf(m[r], sk);
                w = expf(m[r] - M);
                L = l[r] * w + expf(sk - M);
            }
            float rcp = L > 0.f ? w / L : 0.f;
            if (head_gate)
                rcp /= 1.f + expf(-ldf(head_gate + (long)t * hg_tok + h));
            T* o = out + (long)t * out_tok + (long)h * Dv;
#pragma unroll
            for (int i = 0; i < DPL; ++i) {
                const int d = sa_coord<PAIR>(lane, i);
                if (d < Dv) stf(o + d, acc[r][i] * rcp);
            }
        } else {
            const long prow = ((long)split * H + h) * Tn + t;
            if (lane == 0) {
                part_ml[prow * 2] = m[r];
                part_ml[prow * 2 + 1] = l[r];
            }
#pragma unroll
            for (int i = 0; i < DPL; ++i) {
                const int d = sa_coord<PAIR>(lane, i);
                if (d < Dv) part_acc[prow * Dv + d] = acc[r][i];
            }
        }
    }
}

}  // namespace

#define MS_LAUNCH(N, R, P)                                                    \
    mixed_score_pv_kernel<TT, N, R, P>                                        \
        <<<grid, SA_WAVES * WAVE, smem2, s>>>(                                \
            scores, ctx, mix, (const TT*)v_cache, block_table, bt_stride,     \
            positions, seq_idx, sink, (TT*)out, out_tok, part_acc, part_ml,   \
            Tn, H, G, Dv, bs, window, (const TT*)head_gate, hg_tok)

#define MS_CASE(N, P)                                                         \
    if (dpl == N && pair == P) {                                              \
        if (rep == 4) MS_LAUNCH(N, 4, P);                                     \
        else if (rep == 2) MS_LAUNCH(N, 2, P);                                \
        else MS_LAUNCH(N, 1, P);                                              \
        launched = true;                                                      \
    }

template <typename TT>
static int mixed_score_dispatch(const void* q, long q_tok, const void* k_cache,
                                const void* v_cache, const int* block_table,
                                int bt_stride, const int* positions,
                                const int* seq_idx, float softcap,
                                const float* mix, const float* sink,
                                const void* head_gate, long hg_tok, void* out,
                                long out_tok, float* scores, long ctx,
                                float* scratch_ml, float* part_acc,
                                float* part_ml, int splits, int Tn, int H,
                                int G, int D, int Dv, int bs, int window,
                                hipStream_t s) {
    const bool pair = Dv % 2 == 0;
    int dpl = pair ? 2 * ((Dv + 2 * WAVE - 1) / (2 * WAVE))
                   : (Dv + WAVE - 1) / WAVE;
    if (dpl == 3) dpl = 4;
    const int group = H / G;
    const int rep = group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1;
    const int units = H / rep;
    const dim3 grid(Tn, (units + SA_WAVES - 1) / SA_WAVES, splits);
    const size_t smem1 = (size_t)SA_WAVES * rep * D * sizeof(float);
    const size_t smem2 = (size_t)SA_WAVES * rep * H * sizeof(float);
#define TS_LAUNCH(R)                                                          \
    talk_scores_kernel<TT, R><<<grid, SA_WAVES * WAVE, smem1, s>>>(           \
        (const TT*)q, q_tok, (const TT*)k_cache, block_table, bt_stride,      \
        positions, seq_idx, scores, ctx, scratch_ml, Tn, H, G, D, bs, window, \
        softcap)
    if (rep == 4) TS_LAUNCH(4);
    else if (rep == 2) TS_LAUNCH(2);
    else TS_LAUNCH(1);
#undef TS_LAUNCH
    bool launched = false;
    MS_CASE(2, true) MS_CASE(4, true)
    MS_CASE(1, false) MS_CASE(2, false) MS_CASE(4, false)
    if (!launched) return 1;
    if (splits > 1) {
        const dim3 g2(Tn, (H + SA_WAVES - 1) / SA_WAVES);
        sink_attn_combine_kernel<TT><<<g2, SA_WAVES * WAVE, 0, s>>>(
            part_acc, part_ml, sink, (TT*)out, out_tok, 1.f, splits, Tn, H, Dv,
            (const TT*)head_gate, hg_tok);
    }
    return 0;
}

// scores [Tn, H, ctx] fp32 (ctx >= the longest visible key range);
// scratch_ml [splits, Tn, H, 2] (per-split statistics of the unmixed scores,
// unused); part_acc [splits, H, Tn, Dv], part_ml [splits, H, Tn, 2] (unused
// when splits == 1). mix fp32 [H, H]; softcap 0: no cap. Nonzero when a head
// size exceeds 256.
extern "C" int launch_mixed_score_attn(
    const void* q, long q_tok, const void* k_cache, const void* v_cache,
    const int* block_table, int bt_stride, const int* positions,
    const int* seq_idx, float softcap, const float* mix, const float* sink,
    const void* head_gate, long hg_tok, void* out, long out_tok, float* scores,
    long ctx, float* scratch_ml, float* part_acc, float* part_ml, int splits,
    int Tn, int H, int G, int D, int Dv, int bs, int window, int f32,
    hipStream_t s) {
    if (D > SA_MAXD || Dv > SA_MAXD) return 1;
    if (Tn == 0) return 0;
    if (f32)
        return mixed_score_dispatch<float>(
            q, q_tok, k_cache, v_cache, block_table, bt_stride, positions,
            seq_idx, softcap, mix, sink, head_gate, hg_tok, out, out_tok,
            scores, ctx, scratch_ml, part_acc, part_ml, splits, Tn, H, G, D,
            Dv, bs, window, s);
    return mixed_score_dispatch<unsigned short>(
        q, q_tok, k_cache, v_cache, block_table, bt_stride, positions,
        seq_idx, softcap, mix, sink, head_gate, hg_tok, out, out_tok, scores,
        ctx, scratch_ml, part_acc, part_ml, splits, Tn, H, G, D, Dv, bs,
        window, s);
}
