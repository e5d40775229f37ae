// Varlen causal prefill attention (flash-style, no S x S materialization).
//
// Both kernels are templated over PAGED: when true, K/V come from the paged
// KV cache ([nb, nkv, bs, hd] + block table) instead of the packed fresh
// projections, and each query chunk attends to the full cached history
// (chunked prefill: query row j of sequence b has absolute position
// hist + j where hist = seq_lens[b] - query_len[b]). The chunk's own K/V
// were stored to the cache by kv_store before this kernel runs.
//
// Two kernels:
//  * attn_prefill_mfma — the production path for head_dim 64/128: per
//    workgroup 4 waves x 16 q-rows (64-row Q tile), 32-key K/V tiles staged
//    in LDS (+8-element row padding => conflict-free ds_read_b128, guide
//    T2/G4), QK^T and P.V on v_mfma_f32_16x16x32_bf16, online softmax in
//    registers with a 16-lane-group shuffle reduce, V transposed at staging
//    so the PV B-fragment is a contiguous 16 B LDS read.
//  * attn_prefill_basic — correctness fallback for small/odd head dims
//    (test models): per (seq, head) workgroup, lanes-over-keys scores +
//    lanes-over-dims PV like the decode kernel.
//
// Numerics reference: ops/reference.py attn_prefill.
#include "common.h"

// KV element loaders shared by the bf16 and fp8 (OCP e4m3) cache paths
__device__ __forceinline__ float kv_elem_f32(unsigned short x) {
    return bf2f(x);
}
__device__ __forceinline__ float kv_elem_f32(unsigned char x) {
    return fp8x2_2f((unsigned short)x).x;
}
__device__ __forceinline__ bf16x8 load_kv8_bf16(const unsigned short* p) {
    return *reinterpret_cast<const bf16x8*>(p);
}
__device__ __forceinline__ bf16x8 load_kv8_bf16(const unsigned char* p) {
    float f[8];
    load_fp8x8(p, f);
    bf16x8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (__bf16)f[e];
    return r;
}

// ------------------------------------------------------------------ basic
template <bool PAGED, typename KVT>
__global__ __launch_bounds__(64) void attn_prefill_basic(
    const unsigned short* __restrict__ q,  // [T, nq, hd]
    const KVT* __restrict__ k,  // [T,nkv,hd] | PAGED: [nb,nkv,bs,hd]
    const KVT* __restrict__ v,
    const int* __restrict__ cu,            // [nseq+1] (query tokens)
    const int* __restrict__ block_table,   // PAGED only: [nseq, W]
    const int* __restrict__ seq_lens,      // PAGED only: total len incl chunk
    unsigned short* __restrict__ out,      // [T, nq, hd]
    int nq, int nkv, int hd, long s_q, long s_k, long s_v, int W, int bs,
    float scale, int causal) {
    const int seq = blockIdx.y;
    const int h = blockIdx.x;
    const int kvh = h / (nq / nkv);
    const int s0 = cu[seq], s1 = cu[seq + 1];
    const int QL = s1 - s0;
    const int L = PAGED ? seq_lens[seq] : QL;
    const int hist = L - QL;
    const int* bt = PAGED ? block_table + (long)seq * W : nullptr;
    const int lane = threadIdx.x;

    extern __shared__ __attribute__((aligned(16))) char smem_raw[];
    float* q_s = reinterpret_cast<float*>(smem_raw);  // [hd]
    float* p_s = q_s + hd;                            // [WAVE]

    for (int r = 0; r < QL; ++r) {  // one q row at a time
        for (int d = lane; d < hd; d += WAVE)
            q_s[d] = bf2f(q[(long)(s0 + r) * s_q + (long)h * hd + d]) * scale;
        __builtin_amdgcn_s_barrier();
        const int kmax = causal ? hist + r + 1 : L;
        float m = -1e30f, lsum = 0.f, o0 = 0.f, o1 = 0.f;
        const int d0 = lane * 2;
        for (int base = 0; base < kmax; base += WAVE) {
            const int key = base + lane;
            float s = -1e30f;
            if (key < kmax) {
                s = 0.f;
                const KVT* kr;
                if (PAGED)
                    kr = k + (((long)bt[key / bs] * nkv + kvh) * bs +
                              key % bs) * hd;
                else
                    kr = k + (long)(s0 + key) * s_k + (long)kvh * hd;
                for (int d = 0; d < hd; ++d)
                    s = fmaf(kv_elem_f32(kr[d]), q_s[d], s);
            }
            float cmax = wave_max(s);
            float mn = fmaxf(m, cmax);
            float p = (key < kmax) ? __expf(s - mn) : 0.f;
            float alpha = __expf(m - mn);
            m = mn;
            lsum = lsum * alpha + wave_sum(p);
            o0 *= alpha;
            o1 *= alpha;
            p_s[lane] = p;
            const int nk = min(WAVE, kmax - base);
            if (d0 < hd) {
                for (int t = 0; t < nk; ++t) {
                    const int vk = base + t;
                    const KVT* vr;
                    if (PAGED)
                        vr = v + (((long)bt[vk / bs] * nkv + kvh) * bs +
                                  vk % bs) * hd;
                    else
                        vr = v + (long)(s0 + vk) * s_v + (long)kvh * hd;
                    o0 = fmaf(p_s[t], kv_elem_f32(vr[d0]), o0);
                    o1 = fmaf(p_s[t], kv_elem_f32(vr[d0 + 1]), o1);
                }
            }
        }
        if (d0 < hd) {
            const float inv = (lsum > 0.f) ? 1.f / lsum : 0.f;
            unsigned short* orow = out + ((long)(s0 + r) * nq + h) * hd;
            orow[d0] = f2bf(o0 * inv);
            orow[d0 + 1] = f2bf(o1 * inv);
        }
        __builtin_amdgcn_s_barrier();
    }
}

// ------------------------------------------------------------------- mfma
// Fragment maps for v_mfma_f32_16x16x32_bf16 (gfx950):
//   A (16x32): lane holds row (l&15), k = (l>>4)*8 + e   (8 bf16)
//   B (32x16): lane holds col (l&15), k = (l>>4)*8 + e   (8 bf16)
//   C (16x16): lane holds col (l&15), rows (l>>4)*4 + r  (4 f32)
// Verified on hardware by tests/test_ops_gpu.py::test_mfma_fragment_map.
#define PF_QROWS 16   // q rows per wave
#define PF_WAVES 4
#define PF_TM (PF_QROWS * PF_WAVES)  // 64-row q tile per workgroup
#define PF_TN 64                     // kv tile (4 x 16-key fragments)
#define PF_PAD 8                     // LDS row padding (bf16 elems)

// HILO: the softmax weights enter the P V product as a bf16 PAIR (hi + lo,
// two MFMAs, ~16 mantissa bits) instead of one bf16 rounding — for designs
// whose attention weights are 32-bit quantities. sink (optional, [nq] fp32):
// a per-head logit counted once in the softmax denominator, with no key and
// no value. The output row of token t, head h starts at out + t*s_o + h*HD
// and is multiplied by out_scale. window > 0: the row at absolute position
// p sees keys p - window < j <= p, and key tiles wholly before the tile's
// first window are skipped. head_gate (optional, bf16 [tokens, nq] with row
// stride s_g): head h's output times sigmoid(head_gate[t, h]).
//
// MODE 1 / MODE 2 split the kernel around a score buffer, for attention
// whose scores are mixed across heads before the softmax: MODE 1 stops
// after S = Q K^T, caps it (softcap > 0: softcap * tanh(s / softcap)) and
// writes the tile — masked entries too, as they come — to score_buf; MODE
// 2 takes its score tiles from score_buf instead of computing them (another
// kernel has mixed the heads in between) and goes on with mask, softmax,
// P V and the epilogue. score_buf [nseq, qt_rows, nq, ctx] fp32 holds the
// query rows [qt0 * 64, qt0 * 64 + qt_rows) of every chunk; entry `col` of
// a row is key kv_lo + col, kv_lo being the first key the row's 64-query
// tile visits. blockIdx.x counts tiles from qt0.
template <int HD, bool PAGED, typename KVT, bool HILO = false, int MODE = 0>
__global__ __launch_bounds__(256) void attn_prefill_mfma(
    const unsigned short* __restrict__ q,
    const KVT* __restrict__ k,  // PAGED: k_cache [nb,nkv,bs,hd]
    const KVT* __restrict__ v,
    const int* __restrict__ cu,            // [nseq+1] query tokens
    const int* __restrict__ block_table,   // PAGED only
    const int* __restrict__ seq_lens,      // PAGED only
    unsigned short* __restrict__ out,
    int nq, int nkv, long s_q, long s_k, long s_v, int W, int bs,
    float scale, const float* __restrict__ sink, float out_scale, long s_o,
    int window = 0, const unsigned short* __restrict__ head_gate = nullptr,
    long s_g = 0, float* __restrict__ score_buf = nullptr, int qt0 = 0,
    int qt_rows = 0, long ctx = 0, float softcap = 0.f) {
    constexpr int KSTEPS = HD / 32;
    const int seq = blockIdx.z;
    const int h = blockIdx.y;
    const int kvh = h / (nq / nkv);
    const int s0 = cu[seq], s1 = cu[seq + 1];
    const int QL = s1 - s0;                // query rows in this chunk
    const int L = PAGED ? seq_lens[seq] : QL;  // keys incl. cached history
    const int hist = L - QL;
    const int* bt = PAGED ? block_table + (long)seq * W : nullptr;
    const int q0 = (blockIdx.x + qt0) * PF_TM;  // q tile base (chunk-local row)
    if (q0 >= QL) return;

    const int tid = threadIdx.x;
    const int lane = tid % WAVE;
    const int wid = tid / WAVE;
    const int lg = lane >> 4;   // 4 lane groups of 16
    const int li = lane & 15;

    extern __shared__ __attribute__((aligned(16))) char smem_raw[];
    // K tile [PF_TN][HD+PAD], V^T tile [HD][PF_TN+PAD], both bf16.
    // The K buffer is later reused as the P tile [PF_TM][PF_TN+PAD], so the
    // V^T carve starts past max(K tile, P tile) — at HD=64 the P tile is the
    // larger one and a K-sized carve would let P overwrite V^T.
    constexpr int VT_STRIDE = PF_TN + PF_PAD;
    constexpr int K_ELEMS = PF_TN * (HD + PF_PAD);
    constexpr int P_TILE = PF_TM * VT_STRIDE;
    constexpr int P_ELEMS = P_TILE * (HILO ? 2 : 1);
    constexpr int VT_OFF = (K_ELEMS > P_ELEMS ? K_ELEMS : P_ELEMS);
    unsigned short* k_s = reinterpret_cast<unsigned short*>(smem_raw);
    unsigned short* vt_s = k_s + VT_OFF;

    // ---- load this wave's Q rows into A-fragments (registers), scaled
    bf16x8 a_q[KSTEPS];
    const int my_qrow = q0 + wid * PF_QROWS + li;  // A row = li
    const bool row_ok = my_qrow < QL;
    if (MODE != 2) {
        const unsigned short* qr = q + (long)(s0 + my_qrow) * s_q + (long)h * HD;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const int d = ks * 32 + lg * 8;
            if (row_ok) {
                short8 raw = *reinterpret_cast<const short8*>(qr + d);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    a_q[ks][e] = (__bf16)(bf2f((unsigned short)raw[e]) * scale);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) a_q[ks][e] = (__bf16)0.f;
            }
        }
    }

    // online softmax state: this lane covers rows (lg*4 + r) of the wave's
    // 16-row block; stats per C-row slot r (4 rows), kept redundantly by
    // the 16 lanes of each group.
    float m_run[4], l_run[4];
    f32x4 o_acc[HD / 16];  // C frags: [dim block][4 rows]
#pragma unroll
    for (int r = 0; r < 4; ++r) { m_run[r] = -1e30f; l_run[r] = 0.f; }
#pragma unroll
    for (int nb = 0; nb < HD / 16; ++nb) o_acc[nb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // causal: keys up to the last absolute q position of this tile
    const int kv_end = min(L, hist + q0 + PF_TM);
    // window: the tile's first row is the one that reaches back farthest
    const int kv_lo =
        window > 0 ? max(0, hist + q0 - window + 1) / PF_TN * PF_TN : 0;

    for (int kb = kv_lo; kb < kv_end; kb += PF_TN) {
        // ---- stage K tile [32][HD] and V^T tile [HD][32]
        __syncthreads();
        {
            // each thread loads 16 B: key = tid / (HD/8), dims 8*(tid % ...)
            constexpr int THREADS_PER_ROW = HD / 8;
            for (int i = tid; i < PF_TN * THREADS_PER_ROW; i += 256) {
                const int key = i / THREADS_PER_ROW;
                const int d = (i % THREADS_PER_ROW) * 8;
                const int gk = kb + key;
                bf16x8 kraw{}, vraw{};
                if (gk < kv_end) {
                    if (PAGED) {
                        const long koff = (((long)bt[gk / bs] * nkv + kvh) *
                                           bs + gk % bs) * HD + d;
                        if (MODE != 2) kraw = load_kv8_bf16(k + koff);
                        if (MODE != 1) vraw = load_kv8_bf16(v + koff);
                    } else {
                        kraw = load_kv8_bf16(
                            k + (long)(s0 + gk) * s_k + (long)kvh * HD + d);
                        vraw = load_kv8_bf16(
                            v + (long)(s0 + gk) * s_v + (long)kvh * HD + d);
                    }
                }
                if (MODE != 2)
                    *reinterpret_cast<bf16x8*>(k_s + key * (HD + PF_PAD) + d) =
                        kraw;
                if (MODE != 1) {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        vt_s[(d + e) * VT_STRIDE + key] =
                            ((const unsigned short*)&vraw)[e];
                }
            }
        }
        __syncthreads();

        // ---- S = Q K^T : PF_TN/16 16-key column fragments
        f32x4 sfrag[PF_TN / 16];
        if (MODE == 2) {
            // the (head-mixed) scores of this tile, C layout: col li, rows
            // lg*4 + r
#pragma unroll
            for (int f = 0; f < PF_TN / 16; ++f)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int qrow = q0 + wid * PF_QROWS + lg * 4 + r;
                    float sv = 0.f;
                    if (qrow < QL)
                        sv = score_buf[(((long)seq * qt_rows +
                                         (qrow - qt0 * PF_TM)) * nq + h) * ctx +
                                       (kb - kv_lo + f * 16 + li)];
                    sfrag[f][r] = sv;
                }
        } else {
#pragma unroll
            for (int f = 0; f < PF_TN / 16; ++f) {
                f32x4 acc{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ++ks) {
                    // B-frag: col = key (li + 16f), k = dim ks*32 + lg*8 + e
                    bf16x8 bk = *reinterpret_cast<const bf16x8*>(
                        k_s + (f * 16 + li) * (HD + PF_PAD) + ks * 32 + lg * 8);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        a_q[ks], bk, acc, 0, 0, 0);
                }
                sfrag[f] = acc;
            }
        }
        if (MODE == 1) {
#pragma unroll
            for (int f = 0; f < PF_TN / 16; ++f)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int qrow = q0 + wid * PF_QROWS + lg * 4 + r;
                    float sv = sfrag[f][r];
                    if (softcap > 0.f) sv = softcap * tanhf(sv / softcap);
                    if (qrow < QL)
                        score_buf[(((long)seq * qt_rows +
                                    (qrow - qt0 * PF_TM)) * nq + h) * ctx +
                                  (kb - kv_lo + f * 16 + li)] = sv;
                }
            continue;       // the barrier at the loop head guards k_s
        }

        // ---- causal mask + online softmax (rows rr = lg*4 + r)
        float pmax[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) pmax[r] = -1e30f;
#pragma unroll
        for (int f = 0; f < PF_TN / 16; ++f) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int qrow = q0 + wid * PF_QROWS + lg * 4 + r;
                const int key = kb + f * 16 + li;
                if (key > hist + qrow || qrow >= QL || key >= kv_end ||
                    (window > 0 && key <= hist + qrow - window))
                    sfrag[f][r] = -1e30f;
                pmax[r] = fmaxf(pmax[r], sfrag[f][r]);
            }
        }
        // row max across the 16 lanes of the group (cols)
#pragma unroll
        for (int off = 1; off < 16; off <<= 1)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                pmax[r] = fmaxf(pmax[r], __shfl_xor(pmax[r], off));

        float alpha[4], psum[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float mn = fmaxf(m_run[r], pmax[r]);
            alpha[r] = __expf(m_run[r] - mn);
            m_run[r] = mn;
            psum[r] = 0.f;
        }
        // P = exp(S - m); convert to bf16 A-fragment via LDS staging:
        // reuse k_s as the P tile [PF_TM][PF_TN+PAD] (barrier-protected).
        unsigned short* p_s = k_s;  // reuse; careful with sizes (TM*(TN+8))
        __syncthreads();  // everyone done reading K before overwrite
#pragma unroll
        for (int f = 0; f < PF_TN / 16; ++f) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float pv = __expf(sfrag[f][r] - m_run[r]);
                if (sfrag[f][r] <= -1e29f) pv = 0.f;
                psum[r] += pv;
                const int pi =
                    (wid * PF_QROWS + lg * 4 + r) * VT_STRIDE + f * 16 + li;
                const unsigned short hi = f2bf(pv);
                p_s[pi] = hi;
                if (HILO) p_s[P_TILE + pi] = f2bf(pv - bf2f(hi));
            }
        }
        // row sum across group lanes
#pragma unroll
        for (int off = 1; off < 16; off <<= 1)
#pragma unroll
            for (int r = 0; r < 4; ++r) psum[r] += __shfl_xor(psum[r], off);
#pragma unroll
        for (int r = 0; r < 4; ++r)
            l_run[r] = l_run[r] * alpha[r] + psum[r];

        // rescale O by alpha (alpha is per C-row r, uniform across cols)
#pragma unroll
        for (int nb = 0; nb < HD / 16; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) o_acc[nb][r] *= alpha[r];

        // ---- O += P V : A = P rows of this wave, B = V^T
        // (p_s writes above are within-wave for our rows; but other waves
        // share the LDS buffer -> sync so K-tile reuse is safe)
        __syncthreads();
        bf16x8 a_p[PF_TN / 32];  // A k-dim = keys: 32 keys per fragment
        bf16x8 a_pl[HILO ? PF_TN / 32 : 1];
#pragma unroll
        for (int ks2 = 0; ks2 < PF_TN / 32; ++ks2) {
            const int pi = (wid * PF_QROWS + li) * VT_STRIDE + ks2 * 32 + lg * 8;
            a_p[ks2] = *reinterpret_cast<const bf16x8*>(p_s + pi);
            if (HILO)
                a_pl[ks2] = *reinterpret_cast<const bf16x8*>(p_s + P_TILE + pi);
        }
#pragma unroll
        for (int nb = 0; nb < HD / 16; ++nb) {
#pragma unroll
            for (int ks2 = 0; ks2 < PF_TN / 32; ++ks2) {
                bf16x8 bv = *reinterpret_cast<const bf16x8*>(
                    vt_s + (nb * 16 + li) * VT_STRIDE + ks2 * 32 + lg * 8);
                o_acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    a_p[ks2], bv, o_acc[nb], 0, 0, 0);
                if (HILO)
                    o_acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        a_pl[ks2], bv, o_acc[nb], 0, 0, 0);
            }
        }
    }

    if (MODE == 1) return;
    // ---- epilogue: normalize and store (C layout: col=li, row=lg*4+r)
    const int orow_base = q0 + wid * PF_QROWS;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int qrow = orow_base + lg * 4 + r;
        if (qrow >= QL) continue;
        float lsum = l_run[r], w = out_scale;
        if (sink) {
            const float sk = sink[h];
            const float M = fmaxf(m_run[r], sk);
            const float e = __expf(m_run[r] - M);
            lsum = lsum * e + __expf(sk - M);
            w *= e;
        }
        if (head_gate)
            w /= 1.f + __expf(-bf2f(head_gate[(long)(s0 + qrow) * s_g + h]));
        const float inv = (lsum > 0.f) ? w / lsum : 0.f;
        unsigned short* orow = out + (long)(s0 + qrow) * s_o + (long)h * HD;
#pragma unroll
        for (int nb = 0; nb < HD / 16; ++nb)
            orow[nb * 16 + li] = f2bf(o_acc[nb][r] * inv);
    }
}

static int prefill_mfma_smem(int hd, int hilo = 0) {
    // LDS: max(K tile, P tile(s)) + V^T tile, bf16; must match VT_OFF
    const int k_bytes = PF_TN * (hd + PF_PAD) * 2;
    const int p_bytes = PF_TM * (PF_TN + PF_PAD) * 2 * (hilo ? 2 : 1);
    const int vt_bytes = hd * (PF_TN + PF_PAD) * 2;
    return (k_bytes > p_bytes ? k_bytes : p_bytes) + vt_bytes;
}

extern "C" void launch_attn_prefill(
    const unsigned short* q, const unsigned short* k, const unsigned short* v,
    const int* cu, unsigned short* out, int nseq, int nq, int nkv, int hd,
    long s_q, long s_k, long s_v, int max_seqlen, float scale, int causal,
    hipStream_t stream) {
    if ((hd == 64 || hd == 128) && causal) {
        const int tiles = (max_seqlen + PF_TM - 1) / PF_TM;
        dim3 grid(tiles, nq, nseq);
        const int smem = prefill_mfma_smem(hd);
        if (hd == 128)
            hipLaunchKernelGGL((attn_prefill_mfma<128, false, unsigned short>),
                               grid, dim3(256), smem, stream, q, k, v, cu,
                               nullptr, nullptr, out, nq, nkv, s_q, s_k, s_v,
                               0, 0, scale, nullptr, 1.f, (long)nq * hd);
        else
            hipLaunchKernelGGL((attn_prefill_mfma<64, false, unsigned short>),
                               grid, dim3(256), smem, stream, q, k, v, cu,
                               nullptr, nullptr, out, nq, nkv, s_q, s_k, s_v,
                               0, 0, scale, nullptr, 1.f, (long)nq * hd);
        return;
    }
    dim3 grid(nq, nseq);
    const int smem = (hd + WAVE) * 4;
    hipLaunchKernelGGL((attn_prefill_basic<false, unsigned short>), grid,
                       dim3(WAVE), smem, stream, q, k, v, cu, nullptr,
                       nullptr, out, nq, nkv, hd, s_q, s_k, s_v, 0, 0, scale,
                       causal);
}

// Chunked prefill: query chunks (packed varlen, cu) attend to the full
// paged history; the chunk's K/V are already in the cache (kv_store ran
// first), so K/V come exclusively from the paged pool.
extern "C" void launch_attn_prefill_paged(
    const unsigned short* q, const void* k_cache, const void* v_cache,
    const int* cu, const int* block_table, const int* seq_lens,
    unsigned short* out, int nseq, int nq, int nkv, int hd, long s_q, int W,
    int bs, int max_qlen, float scale, int fp8, hipStream_t stream) {
#define PFP_LAUNCH(KVT)                                                        \
    do {                                                                       \
        const KVT* kc = reinterpret_cast<const KVT*>(k_cache);                 \
        const KVT* vc = reinterpret_cast<const KVT*>(v_cache);                 \
        if (hd == 64 || hd == 128) {                                           \
            const int tiles = (max_qlen + PF_TM - 1) / PF_TM;                  \
            dim3 grid(tiles, nq, nseq);                                        \
            const int smem = prefill_mfma_smem(hd);                            \
            if (hd == 128)                                                     \
                hipLaunchKernelGGL((attn_prefill_mfma<128, true, KVT>), grid,  \
                                   dim3(256), smem, stream, q, kc, vc, cu,     \
                                   block_table, seq_lens, out, nq, nkv, s_q,   \
                                   0, 0, W, bs, scale, nullptr, 1.f,           \
                                   (long)nq * hd);                             \
            else                                                               \
                hipLaunchKernelGGL((attn_prefill_mfma<64, true, KVT>), grid,   \
                                   dim3(256), smem, stream, q, kc, vc, cu,     \
                                   block_table, seq_lens, out, nq, nkv, s_q,   \
                                   0, 0, W, bs, scale, nullptr, 1.f,           \
                                   (long)nq * hd);                             \
            return;                                                            \
        }                                                                      \
        dim3 grid(nq, nseq);                                                   \
        const int smem = (hd + WAVE) * 4;                                      \
        hipLaunchKernelGGL((attn_prefill_basic<true, KVT>), grid, dim3(WAVE),  \
                           smem, stream, q, kc, vc, cu, block_table, seq_lens, \
                           out, nq, nkv, hd, s_q, 0, 0, W, bs, scale, 1);      \
    } while (0)
    if (fp8) PFP_LAUNCH(unsigned char);
    else PFP_LAUNCH(unsigned short);
#undef PFP_LAUNCH
}

// Packed query chunks against the paged history with fp32-grade softmax
// weights (bf16 hi+lo pair), an optional per-head sink logit, an output
// scale and a strided output (a column slice of a wider buffer). bf16,
// head size 64 or 128 (returns nonzero otherwise); scale is applied by the
// caller (folded into q). window 0: causal without a window; head_gate
// optional (see the kernel).
extern "C" int launch_attn_prefill_paged_sink(
    const unsigned short* q, long s_q, const unsigned short* k_cache,
    const unsigned short* v_cache, const int* cu, const int* block_table,
    const int* seq_lens, unsigned short* out, long s_o, int nseq, int nq,
    int nkv, int hd, int W, int bs, int max_qlen, const float* sink,
    float out_scale, int window, const unsigned short* head_gate, long s_g,
    hipStream_t stream) {
    if (hd != 64 && hd != 128) return 1;
    if (nseq == 0 || max_qlen == 0) return 0;
    const int tiles = (max_qlen + PF_TM - 1) / PF_TM;
    dim3 grid(tiles, nq, nseq);
    const int smem = prefill_mfma_smem(hd, 1);
    if (hd == 128)
        hipLaunchKernelGGL(
            (attn_prefill_mfma<128, true, unsigned short, true>), grid,
            dim3(256), smem, stream, q, k_cache, v_cache, cu, block_table,
            seq_lens, out, nq, nkv, s_q, 0, 0, W, bs, 1.f, sink, out_scale,
            s_o, window, head_gate, s_g);
    else
        hipLaunchKernelGGL(
            (attn_prefill_mfma<64, true, unsigned short, true>), grid,
            dim3(256), smem, stream, q, k_cache, v_cache, cu, block_table,
            seq_lens, out, nq, nkv, s_q, 0, 0, W, bs, 1.f, sink, out_scale,
            s_o, window, head_gate, s_g);
    return 0;
}

// ------------------------------------------------- scores mixed across heads
// In place on a score buffer [nseq, qt_rows, nq, ctx] (see attn_prefill_mfma
// MODE 1/2): s'_h = sum_g mix[h, g] s_g at every (row, column) the tile
// kernels visit. Workgroup = SM_ROWS rows x 64 columns; a thread stages the
// nq scores of its (row, column) in LDS, then writes the nq mixtures back to
// the same places (it is their only reader and writer).
constexpr int SM_ROWS = 4;
__global__ __launch_bounds__(64 * SM_ROWS) void score_mix_kernel(
    float* __restrict__ score_buf, const float* __restrict__ mix,
    const int* __restrict__ cu, const int* __restrict__ seq_lens, int nq,
    int qt0, int qt_rows, long ctx, int window) {
    extern __shared__ __attribute__((aligned(16))) float sm_s[];
    float* tk = sm_s;                              // [nq, nq]
    float* col = sm_s + nq * nq + threadIdx.x;     // [nq] at stride blockDim
    for (int i = threadIdx.x; i < nq * nq; i += blockDim.x) tk[i] = mix[i];
    __syncthreads();
    const int seq = blockIdx.z;
    const int lr = blockIdx.y * SM_ROWS + threadIdx.x / 64;
    const int c = blockIdx.x * 64 + threadIdx.x % 64;
    if (lr >= qt_rows) return;
    const int s0 = cu[seq], QL = cu[seq + 1] - s0;
    const int qrow = qt0 * PF_TM + lr;
    if (qrow >= QL) return;
    const int L = seq_lens[seq], hist = L - QL;
    const int q0 = qrow / PF_TM * PF_TM;
    const int kv_end = min(L, hist + q0 + PF_TM);
    const int kv_lo =
        window > 0 ? max(0, hist + q0 - window + 1) / PF_TN * PF_TN : 0;
    if (c >= (kv_end - kv_lo + PF_TN - 1) / PF_TN * PF_TN) return;
    float* p = score_buf + ((long)seq * qt_rows + lr) * nq * ctx + c;
    const int st = blockDim.x;
    for (int g = 0; g < nq; ++g) col[g * st] = p[(long)g * ctx];
    for (int h = 0; h < nq; ++h) {
        float a = 0.f;
        for (int g = 0; g < nq; ++g) a += tk[h * nq + g] * col[g * st];
        p[(long)h * ctx] = a;
    }
}

// Packed query chunks against the paged history with capped scores mixed
// across heads before the softmax: tile scores (MODE 1), the mix, then
// softmax and P V from the mixed tiles (MODE 2; weights as a bf16 hi+lo
// pair, sink and head gate in the epilogue). Covers the 64-query tiles
// [qt0, qt0 + n_tiles) of every chunk; score_buf holds nseq * n_tiles * 64
// * nq * ctx floats. bf16, head size 64 or 128 (nonzero otherwise); scale
// is folded into q by the caller.
extern "C" int launch_attn_prefill_paged_mixed(
    const unsigned short* q, long s_q, const unsigned short* k_cache,
    const unsigned short* v_cache, const int* cu, const int* block_table,
    const int* seq_lens, unsigned short* out, long s_o, int nseq, int nq,
    int nkv, int hd, int W, int bs, int qt0, int n_tiles, float* score_buf,
    long ctx, float softcap, const float* mix, const float* sink, int window,
    const unsigned short* head_gate, long s_g, hipStream_t stream) {
    if (hd != 64 && hd != 128) return 1;
    if (nseq == 0 || n_tiles == 0) return 0;
    const int qt_rows = n_tiles * PF_TM;
    const dim3 grid(n_tiles, nq, nseq);
    const int smem = prefill_mfma_smem(hd, 1);
    const size_t mix_smem =
        ((size_t)nq * nq + (size_t)nq * 64 * SM_ROWS) * sizeof(float);
    if (mix_smem > 64 * 1024) return 1;
    const dim3 mgrid((unsigned)((ctx + 63) / 64),
                     (qt_rows + SM_ROWS - 1) / SM_ROWS, nseq);
#define PM_LAUNCH(HDV, M)                                                     \
    hipLaunchKernelGGL(                                                       \
        (attn_prefill_mfma<HDV, true, unsigned short, true, M>), grid,        \
        dim3(256), smem, stream, q, k_cache, v_cache, cu, block_table,        \
        seq_lens, out, nq, nkv, s_q, 0, 0, W, bs, 1.f, sink, 1.f, s_o,        \
        window, head_gate, s_g, score_buf, qt0, qt_rows, ctx, softcap)
    if (hd == 128) PM_LAUNCH(128, 1); else PM_LAUNCH(64, 1);
    hipLaunchKernelGGL(score_mix_kernel, mgrid, dim3(64 * SM_ROWS), mix_smem,
                       stream, score_buf, mix, cu, seq_lens, nq, qt0, qt_rows,
                       ctx, window);
    if (hd == 128) PM_LAUNCH(128, 2); else PM_LAUNCH(64, 2);
#undef PM_LAUNCH
    return 0;
}

// ---------------------------------------------------------- cross-value mfma
// The paged MFMA prefill kernel for attention whose softmax weights are
// mixed across heads afterwards: every query head's weights (bf16 hi+lo
// pair) are applied to the values of ALL key/value heads, so the mix can
// be taken on the per-(query head, value head) sums:
//   part[t, n, h, :] = sum_j softmax_h(j) v_n(j)      (normalized, fp32).
// Scores use head h's own key head. window > 0: row at absolute position p
// sees keys p - window < j <= p; key tiles wholly before the tile's first
// window are skipped. Same tiling and fragment maps as attn_prefill_mfma;
// the V^T tile is staged once per value head against the same P tile. A
// launch covers the NV value heads from vh0 on (registers hold NV output
// accumulators); more value heads take further launches.
template <int HD, int NV>
__global__ __launch_bounds__(256) void attn_prefill_cross_mfma(
    const unsigned short* __restrict__ q,
    const unsigned short* __restrict__ k,  // k_cache [nb,nkv,bs,HD]
    const unsigned short* __restrict__ v,  // v_cache [nb,nkv,bs,HD]
    const int* __restrict__ cu, const int* __restrict__ block_table,
    const int* __restrict__ seq_lens, float* __restrict__ part, int nq,
    int nkv, int vh0, long s_q, int W, int bs, int window) {
    constexpr int KSTEPS = HD / 32;
    const int seq = blockIdx.z;
    const int h = blockIdx.y;
    const int kvh = h / (nq / nkv);
    const int s0 = cu[seq], s1 = cu[seq + 1];
    const int QL = s1 - s0;
    const int L = seq_lens[seq];
    const int hist = L - QL;
    const int* bt = block_table + (long)seq * W;
    const int q0 = blockIdx.x * PF_TM;
    if (q0 >= QL) return;

    const int tid = threadIdx.x;
    const int lane = tid % WAVE;
    const int wid = tid / WAVE;
    const int lg = lane >> 4;
    const int li = lane & 15;

    extern __shared__ __attribute__((aligned(16))) char smem_raw[];
    constexpr int VT_STRIDE = PF_TN + PF_PAD;
    constexpr int K_ELEMS = PF_TN * (HD + PF_PAD);
    constexpr int P_TILE = PF_TM * VT_STRIDE;
    constexpr int P_ELEMS = P_TILE * 2;
    constexpr int VT_OFF = (K_ELEMS > P_ELEMS ? K_ELEMS : P_ELEMS);
    unsigned short* k_s = reinterpret_cast<unsigned short*>(smem_raw);
    unsigned short* vt_s = k_s + VT_OFF;

    bf16x8 a_q[KSTEPS];
    const int my_qrow = q0 + wid * PF_QROWS + li;
    const bool row_ok = my_qrow < QL;
    {
        const unsigned short* qr = q + (long)(s0 + my_qrow) * s_q + (long)h * HD;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const int d = ks * 32 + lg * 8;
            if (row_ok) {
                a_q[ks] = *reinterpret_cast<const bf16x8*>(qr + d);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) a_q[ks][e] = (__bf16)0.f;
            }
        }
    }

    float m_run[4], l_run[4];
    f32x4 o_acc[NV][HD / 16];
#pragma unroll
    for (int r = 0; r < 4; ++r) { m_run[r] = -1e30f; l_run[r] = 0.f; }
#pragma unroll
    for (int n = 0; n < NV; ++n)
#pragma unroll
        for (int nb = 0; nb < HD / 16; ++nb)
            o_acc[n][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int kv_end = min(L, hist + q0 + PF_TM);
    int kb0 = 0;
    if (window > 0) kb0 = max(0, hist + q0 - window + 1) / PF_TN * PF_TN;
    constexpr int THREADS_PER_ROW = HD / 8;

    // V^T tile [HD][64 keys] of value head vh. The lanes of a wave take 64
    // different keys and the same 8 coordinates: the 2-byte transposing
    // writes of a wave then fall into 32 different LDS banks (with
    // coordinate-fastest lanes every lane of a key hits the same bank,
    // because a row pitch that keeps 16-byte reads aligned is a multiple of
    // the bank count in words).
    auto stage_vt = [&](int vh, int kb) {
        for (int i = tid; i < PF_TN * THREADS_PER_ROW; i += 256) {
            const int key = i % PF_TN;
            const int d = (i / PF_TN) * 8;
            const int gk = kb + key;
            bf16x8 vraw{};
            if (gk < kv_end) {
                const long base = (long)bt[gk / bs] * nkv * bs + gk % bs;
                vraw = load_kv8_bf16(v + (base + (long)vh * bs) * HD + d);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e)
                vt_s[(d + e) * VT_STRIDE + key] =
                    ((const unsigned short*)&vraw)[e];
        }
    };

    for (int kb = kb0; kb < kv_end; kb += PF_TN) {
        // ---- stage K tile [64][HD] (own key head) and V^T of value head vh0
        __syncthreads();
        for (int i = tid; i < PF_TN * THREADS_PER_ROW; i += 256) {
            const int key = i / THREADS_PER_ROW;
            const int d = (i % THREADS_PER_ROW) * 8;
            const int gk = kb + key;
            bf16x8 kraw{};
            if (gk < kv_end) {
                const long base = (long)bt[gk / bs] * nkv * bs + gk % bs;
                kraw = load_kv8_bf16(k + (base + (long)kvh * bs) * HD + d);
            }
            *reinterpret_cast<bf16x8*>(k_s + key * (HD + PF_PAD) + d) = kraw;
        }
        stage_vt(vh0, kb);
        __syncthreads();

        f32x4 sfrag[PF_TN / 16];
#pragma unroll
        for (int f = 0; f < PF_TN / 16; ++f) {
            f32x4 acc{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                bf16x8 bk = *reinterpret_cast<const bf16x8*>(
                    k_s + (f * 16 + li) * (HD + PF_PAD) + ks * 32 + lg * 8);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_q[ks], bk, acc,
                                                              0, 0, 0);
            }
            sfrag[f] = acc;
        }

        float pmax[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) pmax[r] = -1e30f;
#pragma unroll
        for (int f = 0; f < PF_TN / 16; ++f) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int qrow = q0 + wid * PF_QROWS + lg * 4 + r;
                const int key = kb + f * 16 + li;
                const int p = hist + qrow;
                if (key > p || qrow >= QL || key >= kv_end ||
                    (window > 0 && key <= p - window))
                    sfrag[f][r] = -1e30f;
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
            alpha[r] = __expf(m_run[r] - mn);
            m_run[r] = mn;
            psum[r] = 0.f;
        }
        unsigned short* p_s = k_s;  // the K tile becomes the P tiles (hi, lo)
        __syncthreads();
#pragma unroll
        for (int f = 0; f < PF_TN / 16; ++f) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float pv = __expf(sfrag[f][r] - m_run[r]);
                if (sfrag[f][r] <= -1e29f) pv = 0.f;
                psum[r] += pv;
                const int pi =
                    (wid * PF_QROWS + lg * 4 + r) * VT_STRIDE + f * 16 + li;
                const unsigned short hi = f2bf(pv);
                p_s[pi] = hi;
                p_s[P_TILE + pi] = f2bf(pv - bf2f(hi));
            }
        }
#pragma unroll
        for (int off = 1; off < 16; off <<= 1)
#pragma unroll
            for (int r = 0; r < 4; ++r) psum[r] += __shfl_xor(psum[r], off);
#pragma unroll
        for (int r = 0; r < 4; ++r)
            l_run[r] = l_run[r] * alpha[r] + psum[r];
#pragma unroll
        for (int n = 0; n < NV; ++n)
#pragma unroll
            for (int nb = 0; nb < HD / 16; ++nb)
#pragma unroll
                for (int r = 0; r < 4; ++r) o_acc[n][nb][r] *= alpha[r];

        __syncthreads();
        bf16x8 a_p[PF_TN / 32], a_pl[PF_TN / 32];
#pragma unroll
        for (int ks2 = 0; ks2 < PF_TN / 32; ++ks2) {
            const int pi = (wid * PF_QROWS + li) * VT_STRIDE + ks2 * 32 + lg * 8;
            a_p[ks2] = *reinterpret_cast<const bf16x8*>(p_s + pi);
            a_pl[ks2] = *reinterpret_cast<const bf16x8*>(p_s + P_TILE + pi);
        }
#pragma unroll
        for (int n = 0; n < NV; ++n) {
            if (vh0 + n >= nkv) break;      // uniform over the workgroup
            if (n > 0) {
                // every wave is done with the previous value head's tile
                __syncthreads();
                stage_vt(vh0 + n, kb);
                __syncthreads();
            }
#pragma unroll
            for (int nb = 0; nb < HD / 16; ++nb) {
#pragma unroll
                for (int ks2 = 0; ks2 < PF_TN / 32; ++ks2) {
                    bf16x8 bv = *reinterpret_cast<const bf16x8*>(
                        vt_s + (nb * 16 + li) * VT_STRIDE + ks2 * 32 + lg * 8);
                    o_acc[n][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        a_p[ks2], bv, o_acc[n][nb], 0, 0, 0);
                    o_acc[n][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        a_pl[ks2], bv, o_acc[n][nb], 0, 0, 0);
                }
            }
        }
    }

    const int orow_base = q0 + wid * PF_QROWS;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int qrow = orow_base + lg * 4 + r;
        if (qrow >= QL) continue;
        const float inv = (l_run[r] > 0.f) ? 1.f / l_run[r] : 0.f;
#pragma unroll
        for (int n = 0; n < NV; ++n) {
            if (vh0 + n >= nkv) break;
            float* orow =
                part + (((long)(s0 + qrow) * nkv + vh0 + n) * nq + h) * HD;
#pragma unroll
            for (int nb = 0; nb < HD / 16; ++nb)
                orow[nb * 16 + li] = o_acc[n][nb][r] * inv;
        }
    }
}

// Packed bf16 query chunks against the paged history, each query head's
// softmax weights applied to every value head: part [T, nkv, nq, hd] fp32.
// Head size 64 or 128 (returns nonzero otherwise); every score multiplier
// is already in q.
extern "C" int launch_attn_prefill_paged_cross(
    const unsigned short* q, long s_q, const unsigned short* k_cache,
    const unsigned short* v_cache, const int* cu, const int* block_table,
    const int* seq_lens, float* part, int nseq, int nq, int nkv, int hd,
    int W, int bs, int max_qlen, int window, hipStream_t stream) {
    if ((hd != 64 && hd != 128) || nkv < 1) return 1;
    if (nseq == 0 || max_qlen == 0) return 0;
    const int tiles = (max_qlen + PF_TM - 1) / PF_TM;
    dim3 grid(tiles, nq, nseq);
    const int smem = prefill_mfma_smem(hd, 1);
#define PFC(HDV, NVV)                                                          \
    hipLaunchKernelGGL((attn_prefill_cross_mfma<HDV, NVV>), grid, dim3(256),   \
                       smem, stream, q, k_cache, v_cache, cu, block_table,     \
                       seq_lens, part, nq, nkv, vh0, s_q, W, bs, window)
    // up to four value heads per launch (measured: two launches of two,
    // at twice the waves per SIMD, are slower — the scores are recomputed;
    // so is passing the tiles through registers to prefetch the next one —
    // the extra registers cost the two-value-head form a wave per SIMD)
    const int nv = nkv > 2 ? 4 : nkv;
    for (int vh0 = 0; vh0 < nkv; vh0 += nv) {
        if (hd == 128) {
            if (nv == 4) PFC(128, 4);
            else if (nv == 2) PFC(128, 2);
            else PFC(128, 1);
        } else {
            if (nv == 4) PFC(64, 4);
            else if (nv == 2) PFC(64, 2);
            else PFC(64, 1);
        }
    }
#undef PFC
    return 0;
}
