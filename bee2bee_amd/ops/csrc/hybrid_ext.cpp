// Torch bindings for the hybrid-stack kernels (hybrid.hip, mixers.hip).
// Shapes, strides and dtypes are validated here so the kernels index
// without checks. Activations are bf16 or fp32 (the kernels are instantiated
// for both); residual, norm weights and recurrent state are fp32. All entry
// points are hipGraph-capture safe (no sync, no host reads).
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <optional>
#include <vector>

using torch::Tensor;

extern "C" {
void launch_scalar_rmsnorm(const float*, void*, long, int, float, float, int,
                           hipStream_t);
void launch_add_scalar_rmsnorm(float*, const void*, const void*, void*, long,
                               int, float, float, float, int, int,
                               hipStream_t);
void launch_gated_rmsnorm(const float*, const float*, const void*, long,
                          void*, long, int, float, int, hipStream_t);
void launch_clamped_glu(const void*, void*, long, long, float, float, int,
                        hipStream_t);
void launch_canon_conv(const void*, const float*, void*, const int*,
                       const int*, const int*, const int*, void*, long, int,
                       int, int, int, hipStream_t);
void launch_latent_rope_store(void*, long, long, int, const void*, long,
                              const float*, int, int, int, float, const int*,
                              const float*, const float*, void*, const int*,
                              long, int, hipStream_t);
int launch_latent_attn(const void*, const void*, long, long, const void*,
                       long, const void*, const int*, int, const int*,
                       const int*, void*, float*, float*, int, int, int, int,
                       int, int, int, float, int, const float*, hipStream_t);
int launch_latent_attn_mfma(const void*, const void*, long, long, const void*,
                            long, const void*, const int*, int, const int*,
                            const int*, const int*, void*, float*, float*,
                            int, int, int, int, int, int, int, int, int,
                            float, const float*, hipStream_t);
int lightning_segment_tokens();
int launch_lightning(const void*, const void*, const void*, long,
                     const float*, float*, const int*, const int*, const int*,
                     float*, float*, int, int, int, int, int, int, int,
                     const float*, const float*, int, float, hipStream_t);
void launch_short_conv(const void*, long, const float*, void*, const int*,
                       const int*, const int*, const int*, float*, long, int,
                       int, int, int, int, int, hipStream_t);
void launch_add_rmsnorm_w(float*, const void*, const float*, void*, long, int,
                          float, int, int, hipStream_t);
void launch_relu2(const void*, long, void*, long, long, int, int, int,
                  hipStream_t);
void launch_head_gated_norm(const float*, const float*, const void*, long,
                            void*, long, long, int, int, float, int, float,
                            int, hipStream_t);
void launch_delta_gates(float*, long, int, int, const void*, long,
                        const void*, long, const float*, const float*, float*,
                        float*, long, int, int, int, hipStream_t);
int launch_qk_norm_rope_store(void*, long, int, const void*, long, int, int,
                              const float*, const float*, float, int,
                              const int*, const float*, const float*,
                              const float*, void*, void*, int, const int*,
                              long, int, hipStream_t);
int launch_delta_rule(const float*, const float*, long, const float*, long,
                      const float*, const float*, int, float*, const int*,
                      const int*, const int*, float*, int, int, int, int, int,
                      hipStream_t);
int launch_attn_prefill_paged_sink(const unsigned short*, long,
                                   const unsigned short*,
                                   const unsigned short*, const int*,
                                   const int*, const int*, unsigned short*,
                                   long, int, int, int, int, int, int, int,
                                   const float*, float, int,
                                   const unsigned short*, long, hipStream_t);
int launch_sink_attn(const void*, long, const void*, const void*, const int*,
                     int, const int*, const int*, const float*, void*, long,
                     float, float*, float*, int, int, int, int, int, int, int,
                     int, int, const void*, long, hipStream_t);
}

namespace {

inline hipStream_t stream() {
    return at::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
}

// 0 = bf16, 1 = fp32
int act_code(at::ScalarType t, const char* name) {
    TORCH_CHECK(t == torch::kBFloat16 || t == torch::kFloat32, name,
                " must be bf16 or fp32");
    return t == torch::kFloat32 ? 1 : 0;
}

int act_code(const Tensor& t, const char* name) {
    TORCH_CHECK(t.is_cuda(), name, " must be on GPU");
    return act_code(t.scalar_type(), name);
}

void check_f32(const Tensor& t, const char* name) {
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kFloat32 &&
                    t.is_contiguous(),
                name, " must be a contiguous fp32 GPU tensor");
}

void check_i32(const Tensor& t, const char* name) {
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kInt32 &&
                    t.is_contiguous(),
                name, " must be a contiguous int32 GPU tensor");
}

Tensor scalar_rmsnorm(const Tensor& x, double gain, double eps,
                      at::ScalarType out_dtype) {
    check_f32(x, "x");
    TORCH_CHECK(x.dim() == 2);
    const int oc = act_code(out_dtype, "out_dtype");
    Tensor y = torch::empty(x.sizes(), x.options().dtype(out_dtype));
    launch_scalar_rmsnorm(x.data_ptr<float>(), y.data_ptr(), x.size(0),
                          (int)x.size(1), (float)gain, (float)eps, oc,
                          stream());
    return y;
}

std::optional<Tensor> add_scalar_rmsnorm(Tensor& resid, const Tensor& y,
                                         const std::optional<Tensor>& y2,
                                         double post_gain,
                                         std::optional<double> pre_gain,
                                         double eps,
                                         at::ScalarType out_dtype) {
    check_f32(resid, "resid");
    TORCH_CHECK(resid.dim() == 2 && y.sizes() == resid.sizes() &&
                y.is_contiguous());
    const int yc = act_code(y, "y");
    const int oc = act_code(out_dtype, "out_dtype");
    const void* y2p = nullptr;
    if (y2.has_value()) {
        TORCH_CHECK(y2->sizes() == y.sizes() && y2->is_contiguous() &&
                    y2->scalar_type() == y.scalar_type() && y2->is_cuda());
        y2p = y2->data_ptr();
    }
    std::optional<Tensor> out;
    void* op = nullptr;
    if (pre_gain.has_value()) {
        out = torch::empty(resid.sizes(), resid.options().dtype(out_dtype));
        op = out->data_ptr();
    }
    launch_add_scalar_rmsnorm(resid.data_ptr<float>(), y.data_ptr(), y2p, op,
                              resid.size(0), (int)resid.size(1),
                              (float)post_gain,
                              (float)pre_gain.value_or(1.0), (float)eps, yc,
                              oc, stream());
    return out;
}

Tensor gated_rmsnorm(const Tensor& x, const Tensor& w, const Tensor& gate,
                     double eps, at::ScalarType out_dtype) {
    check_f32(x, "x");
    check_f32(w, "w");
    TORCH_CHECK(x.dim() == 2 && w.numel() == x.size(1));
    const int gc = act_code(gate, "gate");
    TORCH_CHECK(gate.scalar_type() == out_dtype,
                "gate and output share the activation dtype");
    TORCH_CHECK(gate.dim() == 2 && gate.size(0) == x.size(0) &&
                gate.size(1) == x.size(1) && gate.stride(1) == 1);
    Tensor y = torch::empty(x.sizes(), x.options().dtype(out_dtype));
    launch_gated_rmsnorm(x.data_ptr<float>(), w.data_ptr<float>(),
                         gate.data_ptr(), gate.stride(0), y.data_ptr(),
                         x.size(0), (int)x.size(1), (float)eps, gc, stream());
    return y;
}

Tensor clamped_glu(const Tensor& gu, double limit, double alpha) {
    const int c = act_code(gu, "gate_up");
    TORCH_CHECK(gu.is_contiguous() && gu.size(-1) % 2 == 0);
    const long I = gu.size(-1) / 2;
    const long rows = gu.numel() / (2 * I);
    auto shape = gu.sizes().vec();
    shape.back() = I;
    Tensor y = torch::empty(shape, gu.options());
    launch_clamped_glu(gu.data_ptr(), y.data_ptr(), rows, I, (float)limit,
                       (float)alpha, c, stream());
    return y;
}

Tensor canon_conv(const Tensor& h, const Tensor& w, Tensor& state,
                  const Tensor& state_slots, const Tensor& cu,
                  const Tensor& seq_idx, const Tensor& positions) {
    const int c = act_code(h, "h");
    check_f32(w, "w");
    check_i32(state_slots, "state_slots");
    check_i32(cu, "cu_seqlens");
    check_i32(seq_idx, "seq_idx");
    check_i32(positions, "positions");
    TORCH_CHECK(h.dim() == 2 && h.is_contiguous());
    const long T = h.size(0);
    const int C = (int)h.size(1), K = (int)w.size(0) - 1;
    TORCH_CHECK(w.dim() == 2 && w.size(1) == C && K >= 0 && K <= 8,
                "conv weight must be [taps, channels] with taps <= 9");
    const int B = (int)cu.numel() - 1;
    TORCH_CHECK(state_slots.numel() == B && seq_idx.numel() == T &&
                positions.numel() == T);
    if (K > 0)
        TORCH_CHECK(state.is_cuda() && state.is_contiguous() &&
                    state.scalar_type() == h.scalar_type() &&
                    state.dim() == 3 && state.size(1) == K &&
                    state.size(2) == C);
    Tensor out = torch::empty_like(h);
    launch_canon_conv(h.data_ptr(), w.data_ptr<float>(),
                      K > 0 ? state.data_ptr() : nullptr,
                      state_slots.data_ptr<int>(), cu.data_ptr<int>(),
                      seq_idx.data_ptr<int>(), positions.data_ptr<int>(),
                      out.data_ptr(), T, B, C, K, c, stream());
    return out;
}

void latent_rope_store(Tensor& q_rot, const Tensor& kv, const Tensor& kv_norm,
                       double eps, int64_t kv_rank, int64_t rope_dims,
                       const Tensor& positions, const Tensor& cos_t,
                       const Tensor& sin_t, Tensor& cache,
                       const Tensor& slot_mapping) {
    const int c = act_code(kv, "kv");
    check_f32(kv_norm, "kv_norm");
    check_f32(cos_t, "cos");
    check_f32(sin_t, "sin");
    check_i32(positions, "positions");
    check_i32(slot_mapping, "slot_mapping");
    TORCH_CHECK(q_rot.is_cuda() && q_rot.scalar_type() == kv.scalar_type() &&
                cache.scalar_type() == kv.scalar_type() && cache.is_cuda());
    TORCH_CHECK(q_rot.dim() == 3 && q_rot.stride(2) == 1);
    TORCH_CHECK(kv.dim() == 2 && kv.stride(1) == 1);
    const long T = kv.size(0);
    const int R = (int)q_rot.size(2), C = (int)kv_rank;
    TORCH_CHECK(kv.size(1) == C + R && q_rot.size(0) == T);
    TORCH_CHECK(kv_norm.numel() == C);
    TORCH_CHECK(rope_dims >= 0 && rope_dims <= R && rope_dims % 2 == 0);
    TORCH_CHECK(cos_t.dim() == 2 && cos_t.size(1) == rope_dims / 2 &&
                sin_t.sizes() == cos_t.sizes());
    TORCH_CHECK(cache.is_contiguous() && cache.dim() == 3 &&
                cache.size(2) == C + R);
    TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
    launch_latent_rope_store(
        q_rot.data_ptr(), q_rot.stride(0), q_rot.stride(1),
        (int)q_rot.size(1), kv.data_ptr(), kv.stride(0),
        kv_norm.data_ptr<float>(), C, R, (int)rope_dims, (float)eps,
        positions.data_ptr<int>(), cos_t.data_ptr<float>(),
        sin_t.data_ptr<float>(), cache.data_ptr(),
        slot_mapping.data_ptr<int>(), T, c, stream());
}

Tensor latent_attn(const Tensor& q_abs, const Tensor& q_rot,
                   const Tensor& gate, const Tensor& cache,
                   const Tensor& block_table, const Tensor& positions,
                   const Tensor& seq_idx, const Tensor& cu, int64_t window,
                   double scale, int64_t max_qlen,
                   const std::optional<Tensor>& sink) {
    const int c = act_code(q_abs, "q_abs");
    check_i32(cu, "cu_seqlens");
    check_i32(block_table, "block_table");
    check_i32(positions, "positions");
    check_i32(seq_idx, "seq_idx");
    TORCH_CHECK(q_abs.dim() == 3 && q_abs.is_contiguous());
    const int H = (int)q_abs.size(0), Tn = (int)q_abs.size(1),
              C = (int)q_abs.size(2);
    TORCH_CHECK(q_rot.is_cuda() && q_rot.scalar_type() == q_abs.scalar_type() &&
                q_rot.dim() == 3 && q_rot.size(0) == Tn &&
                q_rot.size(1) == H && q_rot.stride(2) == 1);
    const int R = (int)q_rot.size(2);
    TORCH_CHECK(gate.is_cuda() && gate.scalar_type() == q_abs.scalar_type() &&
                gate.dim() == 2 && gate.size(0) == Tn && gate.size(1) == H &&
                gate.stride(1) == 1);
    TORCH_CHECK(cache.is_cuda() && cache.scalar_type() == q_abs.scalar_type() &&
                cache.is_contiguous() && cache.dim() == 3 &&
                cache.size(2) == C + R);
    TORCH_CHECK(block_table.dim() == 2 && positions.numel() == Tn &&
                seq_idx.numel() == Tn && window >= 0);
    // window 0: every earlier position (a window no context reaches)
    if (window == 0) window = 1 << 30;
    const float* sk = nullptr;
    if (sink.has_value()) {
        check_f32(*sink, "sink");
        TORCH_CHECK(sink->numel() == H);
        sk = sink->data_ptr<float>();
    }
    Tensor out = torch::empty_like(q_abs);
    // the most keys a row can see
    const long reach =
        std::min<long>(window, block_table.size(1) * cache.size(1));
    auto f32opt = q_abs.options().dtype(torch::kFloat32);
    Tensor part_acc, part_ml;
    float *pa = nullptr, *pm = nullptr;
    auto alloc_parts = [&](long n) {
        part_acc = torch::empty({n, H, Tn, C}, f32opt);
        part_ml = torch::empty({n, H, Tn, 2}, f32opt);
        pa = part_acc.data_ptr<float>();
        pm = part_ml.data_ptr<float>();
    };
    // bf16 prompt portions (16-query tiles) and pure decode steps (16-head
    // tiles, keys split until ~768 workgroups) run on the matrix cores;
    // fp32, short mixed steps and uncovered shapes take the generic kernel
    if (c == 0 && (max_qlen >= 16 || max_qlen == 1) && C % 8 == 0 &&
        R % 8 == 0 && C + R <= 576) {
        long sp = 1;
        if (max_qlen == 1) {
            // one resident round: 3 workgroups fit a CU's LDS, 256 CUs
            sp = 768 / std::max<long>(1, (long)Tn * ((H + 15) / 16));
            sp = std::max<long>(1, std::min<long>({sp, 16, (reach + 63) / 64}));
            if (sp > 1) alloc_parts(sp);
        }
        const int rc = launch_latent_attn_mfma(
            q_abs.data_ptr(), q_rot.data_ptr(), q_rot.stride(0),
            q_rot.stride(1), gate.data_ptr(), gate.stride(0),
            cache.data_ptr(), block_table.data_ptr<int>(),
            (int)block_table.size(1), cu.data_ptr<int>(),
            positions.data_ptr<int>(), seq_idx.data_ptr<int>(),
            out.data_ptr(), pa, pm, (int)sp, Tn, (int)cu.numel() - 1,
            (int)max_qlen, H, C, R, (int)cache.size(1), (int)window,
            (float)scale, sk, stream());
        TORCH_CHECK(rc == 0, "latent_attn: matrix-core path refused a shape "
                             "its guard admitted");
        return out;
    }
    // few rows: split each row's keys over more workgroups until the chip
    // has ~8 waves per SIMD, at least 32 keys per share
    long splits = 8192 / std::max<long>(1, (long)Tn * H);
    splits = std::min<long>({splits, 16, (reach + 31) / 32});
    splits = std::max<long>(splits, 1);
    if (splits > 1) alloc_parts(splits);
    const int rc = launch_latent_attn(
        q_abs.data_ptr(), q_rot.data_ptr(), q_rot.stride(0), q_rot.stride(1),
        gate.data_ptr(), gate.stride(0), cache.data_ptr(),
        block_table.data_ptr<int>(), (int)block_table.size(1),
        positions.data_ptr<int>(), seq_idx.data_ptr<int>(), out.data_ptr(),
        pa, pm, (int)splits, Tn, H, C, R, (int)cache.size(1), (int)window,
        (float)scale, c, sk, stream());
    TORCH_CHECK(rc == 0, "latent_attn: kv_rank + rot_dim must be <= 1024");
    return out;
}

// decayed linear attention; form 0 = silu inputs, form 1 = rotated q/k
Tensor linear_attn_impl(const Tensor& q, const Tensor& k, const Tensor& v,
                        const Tensor& decay, Tensor& state,
                        const Tensor& state_slots, const Tensor& cu,
                        const Tensor& positions, int64_t max_qlen, int form,
                        const float* cos_t, const float* sin_t, int rdims,
                        float k_scale) {
    const int c = act_code(q, "q");
    check_f32(decay, "decay");
    check_f32(state, "state");
    check_i32(state_slots, "state_slots");
    check_i32(cu, "cu_seqlens");
    check_i32(positions, "positions");
    TORCH_CHECK(q.dim() == 3 && k.sizes() == q.sizes() && v.dim() == 3);
    const long T = q.size(0);
    const int H = (int)q.size(1), D = (int)q.size(2), Dv = (int)v.size(2);
    for (const Tensor* t : {&q, &k, &v}) {
        TORCH_CHECK(t->is_cuda() && t->scalar_type() == q.scalar_type() &&
                    t->size(0) == T && t->size(1) == H &&
                    t->stride(2) == 1 &&
                    (T == 1 || t->stride(0) == q.stride(0)) &&
                    t->stride(1) == t->size(2));
    }
    TORCH_CHECK(decay.numel() == H);
    TORCH_CHECK(state.dim() == 4 && state.size(1) == H &&
                state.size(2) == D && state.size(3) == Dv);
    const int B = (int)cu.numel() - 1;
    TORCH_CHECK(state_slots.numel() == B && positions.numel() == T);
    auto f32opt = q.options().dtype(torch::kFloat32);
    Tensor out = torch::empty({T, (long)H * Dv}, f32opt);
    // chunks longer than one segment: segments run in parallel from zero
    // states and a scan carries the true state across them. n_seg bounds
    // the batch's segment count without reading the lengths.
    const long seg = lightning_segment_tokens();
    long n_seg = 0;
    Tensor ws;
    float* wsp = nullptr;
    if (max_qlen > seg) {
        n_seg = T / seg + B;
        ws = torch::empty({n_seg, (long)H, (long)D, (long)Dv}, f32opt);
        wsp = ws.data_ptr<float>();
    }
    const int rc = launch_lightning(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), q.stride(0),
        decay.data_ptr<float>(), state.data_ptr<float>(),
        state_slots.data_ptr<int>(), cu.data_ptr<int>(),
        positions.data_ptr<int>(), out.data_ptr<float>(), wsp, (int)n_seg, B,
        H, D, Dv, c, form, cos_t, sin_t, rdims, k_scale, stream());
    TORCH_CHECK(rc == 0, "linear attention: key dim must be <= 256");
    return out;
}

Tensor lightning_attn(const Tensor& q, const Tensor& k, const Tensor& v,
                      const Tensor& decay, Tensor& state,
                      const Tensor& state_slots, const Tensor& cu,
                      const Tensor& positions, int64_t max_qlen) {
    return linear_attn_impl(q, k, v, decay, state, state_slots, cu, positions,
                            max_qlen, 0, nullptr, nullptr, 0, 1.f);
}

Tensor retention_attn(const Tensor& q, const Tensor& k, const Tensor& v,
                      const Tensor& decay, int64_t rope_dims,
                      const std::optional<Tensor>& cos_t,
                      const std::optional<Tensor>& sin_t, double k_scale,
                      Tensor& state, const Tensor& state_slots,
                      const Tensor& cu, const Tensor& positions,
                      int64_t max_qlen) {
    const float *cp = nullptr, *sp = nullptr;
    TORCH_CHECK(rope_dims >= 0 && rope_dims % 2 == 0 &&
                rope_dims <= q.size(2));
    if (rope_dims > 0) {
        TORCH_CHECK(cos_t.has_value() && sin_t.has_value());
        check_f32(*cos_t, "cos");
        check_f32(*sin_t, "sin");
        TORCH_CHECK(cos_t->dim() == 2 && cos_t->size(1) == rope_dims / 2 &&
                    sin_t->sizes() == cos_t->sizes());
        cp = cos_t->data_ptr<float>();
        sp = sin_t->data_ptr<float>();
    }
    return linear_attn_impl(q, k, v, decay, state, state_slots, cu, positions,
                            max_qlen, 1, cp, sp, (int)rope_dims,
                            (float)k_scale);
}

// ---- parallel-form stacks: ops that read/write column slices in place

// a [T, n] column slice: unit inner stride, any row stride
void check_slice(const Tensor& t, long T, long n, at::ScalarType dt,
                 const char* name) {
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == dt && t.dim() == 2 &&
                    t.size(0) == T && t.size(1) == n &&
                    (n == 1 || t.stride(1) == 1),
                name, ": expected a [", T, ", ", n, "] column slice");
}

bool aligned4(const Tensor& t) {
    return t.size(1) % 4 == 0 && t.stride(0) % 4 == 0 &&
           reinterpret_cast<uintptr_t>(t.data_ptr()) %
                   (4 * t.element_size()) == 0;
}

std::optional<Tensor> add_rmsnorm_f32(Tensor& resid,
                                      const std::optional<Tensor>& y,
                                      const std::optional<Tensor>& w,
                                      double eps, at::ScalarType out_dtype,
                                      bool add) {
    check_f32(resid, "resid");
    TORCH_CHECK(resid.dim() == 2);
    const long T = resid.size(0);
    const int W = (int)resid.size(1);
    const void* yp = nullptr;
    int yc = 1;
    if (add) {
        TORCH_CHECK(y.has_value() && y->sizes() == resid.sizes() &&
                    y->is_contiguous());
        yc = act_code(*y, "y");
        yp = y->data_ptr();
    }
    const int oc = act_code(out_dtype, "out_dtype");
    std::optional<Tensor> out;
    void* op = nullptr;
    const float* wp = nullptr;
    if (w.has_value()) {
        check_f32(*w, "w");
        TORCH_CHECK(w->numel() == W);
        wp = w->data_ptr<float>();
        out = torch::empty(resid.sizes(), resid.options().dtype(out_dtype));
        op = out->data_ptr();
    }
    if (!yp && !op) return out;
    launch_add_rmsnorm_w(resid.data_ptr<float>(), yp, wp, op, T, W,
                         (float)eps, yc, oc, stream());
    return out;
}

void relu2(const Tensor& x, Tensor& out) {
    const int c = act_code(x, "x");
    check_slice(x, x.size(0), x.size(1), x.scalar_type(), "x");
    check_slice(out, x.size(0), x.size(1), x.scalar_type(), "out");
    launch_relu2(x.data_ptr(), x.stride(0), out.data_ptr(), out.stride(0),
                 x.size(0), (int)x.size(1), aligned4(x) && aligned4(out), c,
                 stream());
}

Tensor short_conv(const Tensor& x, const Tensor& w, Tensor& state,
                  const Tensor& state_slots, const Tensor& cu,
                  const Tensor& seq_idx, const Tensor& positions, bool silu) {
    const int c = act_code(x, "x");
    check_f32(w, "w");
    check_i32(state_slots, "state_slots");
    check_i32(cu, "cu_seqlens");
    check_i32(seq_idx, "seq_idx");
    check_i32(positions, "positions");
    TORCH_CHECK(x.dim() == 2);
    const long T = x.size(0);
    const int C = (int)x.size(1), K = (int)w.size(0) - 1;
    check_slice(x, T, C, x.scalar_type(), "x");
    TORCH_CHECK(w.dim() == 2 && w.size(1) == C && K >= 0 && K <= 8,
                "conv weight must be [taps, channels] with taps <= 9");
    const int B = (int)cu.numel() - 1;
    TORCH_CHECK(state_slots.numel() == B && seq_idx.numel() == T &&
                positions.numel() == T);
    if (K > 0)
        TORCH_CHECK(state.is_cuda() && state.is_contiguous() &&
                    state.scalar_type() == x.scalar_type() &&
                    state.dim() == 3 && state.size(1) == K &&
                    state.size(2) == C);
    Tensor out = torch::empty({T, (long)C},
                              x.options().dtype(torch::kFloat32));
    launch_short_conv(x.data_ptr(), x.stride(0), w.data_ptr<float>(),
                      K > 0 ? state.data_ptr() : nullptr,
                      state_slots.data_ptr<int>(), cu.data_ptr<int>(),
                      seq_idx.data_ptr<int>(), positions.data_ptr<int>(),
                      out.data_ptr<float>(), T, B, C, K, silu ? 1 : 0,
                      aligned4(x) ? 1 : 0, c, stream());
    return out;
}

std::vector<Tensor> delta_gates(Tensor& qk, int64_t n_qk_heads, int64_t dim,
                                const Tensor& b, const Tensor& a,
                                const Tensor& dt_bias, const Tensor& rate,
                                bool channel_decay) {
    TORCH_CHECK(qk.is_cuda() && qk.scalar_type() == torch::kFloat32 &&
                qk.dim() == 2 && qk.stride(1) == 1 &&
                qk.size(1) >= 2 * n_qk_heads * dim);
    check_f32(dt_bias, "dt_bias");
    check_f32(rate, "rate");
    const long T = qk.size(0);
    const int H = (int)rate.numel();
    const int per = channel_decay ? (int)dim : 1;
    const int c = act_code(b, "b");
    check_slice(b, T, H, b.scalar_type(), "b");
    check_slice(a, T, (long)H * per, b.scalar_type(), "a");
    TORCH_CHECK(dt_bias.numel() == (long)H * per);
    auto f32opt = qk.options();
    Tensor beta = torch::empty({T, (long)H}, f32opt);
    Tensor g = torch::empty({T, (long)H * per}, f32opt);
    launch_delta_gates(qk.data_ptr<float>(), qk.stride(0), (int)n_qk_heads,
                       (int)dim, b.data_ptr(), b.stride(0), a.data_ptr(),
                       a.stride(0), dt_bias.data_ptr<float>(),
                       rate.data_ptr<float>(), beta.data_ptr<float>(),
                       g.data_ptr<float>(), T, H, per, c, stream());
    return {beta, g};
}

Tensor delta_rule(const Tensor& q, const Tensor& k, const Tensor& v,
                  const Tensor& beta, const Tensor& g, Tensor& state,
                  const Tensor& state_slots, const Tensor& cu,
                  const Tensor& positions) {
    check_f32(beta, "beta");
    check_f32(g, "g");
    check_f32(state, "state");
    check_i32(state_slots, "state_slots");
    check_i32(cu, "cu_seqlens");
    check_i32(positions, "positions");
    TORCH_CHECK(q.dim() == 3 && k.sizes() == q.sizes() && v.dim() == 3);
    const long T = q.size(0);
    const int G = (int)q.size(1), D = (int)q.size(2);
    const int H = (int)v.size(1), Dv = (int)v.size(2);
    for (const Tensor* t : {&q, &k, &v})
        TORCH_CHECK(t->is_cuda() && t->scalar_type() == torch::kFloat32 &&
                    t->size(0) == T && t->stride(2) == 1 &&
                    t->stride(1) == t->size(2));
    TORCH_CHECK(T <= 1 || k.stride(0) == q.stride(0));
    TORCH_CHECK(G >= 1 && H % G == 0);
    TORCH_CHECK(state.dim() == 4 && state.size(1) == H &&
                state.size(2) == D && state.size(3) == Dv);
    const bool chdec = g.size(1) != H;
    TORCH_CHECK(beta.dim() == 2 && beta.size(0) == T && beta.size(1) == H &&
                g.dim() == 2 && g.size(0) == T &&
                g.size(1) == (chdec ? (long)H * D : (long)H));
    const int B = (int)cu.numel() - 1;
    TORCH_CHECK(state_slots.numel() == B && positions.numel() == T);
    Tensor out = torch::empty({T, (long)H, (long)Dv}, beta.options());
    const int rc = launch_delta_rule(
        q.data_ptr<float>(), k.data_ptr<float>(), q.stride(0),
        v.data_ptr<float>(), v.stride(0), beta.data_ptr<float>(),
        g.data_ptr<float>(), chdec ? 1 : 0, state.data_ptr<float>(),
        state_slots.data_ptr<int>(), cu.data_ptr<int>(),
        positions.data_ptr<int>(), out.data_ptr<float>(), B, H, G, D, Dv,
        stream());
    TORCH_CHECK(rc == 0, "delta_rule: key dim must be <= 256");
    return out;
}

void head_gated_norm(const Tensor& o, const std::optional<Tensor>& w,
                     const Tensor& gate, bool sigmoid, double eps,
                     Tensor& out, double out_scale) {
    check_f32(o, "o");
    TORCH_CHECK(o.dim() == 3);
    const long T = o.size(0);
    const int H = (int)o.size(1), Dv = (int)o.size(2);
    const int c = act_code(gate, "gate");
    check_slice(gate, T, (long)H * Dv, gate.scalar_type(), "gate");
    check_slice(out, T, (long)H * Dv, gate.scalar_type(), "out");
    const float* wp = nullptr;
    if (w.has_value()) {
        check_f32(*w, "w");
        TORCH_CHECK(w->numel() == Dv);
        wp = w->data_ptr<float>();
    }
    launch_head_gated_norm(o.data_ptr<float>(), wp, gate.data_ptr(),
                           gate.stride(0), out.data_ptr(), out.stride(0), T,
                           H, Dv, (float)eps, sigmoid ? 1 : 0,
                           (float)out_scale, c, stream());
}

void qk_norm_rope_store(Tensor& q, const Tensor& k, const Tensor& q_norm,
                        const Tensor& k_norm, double eps, int64_t rope_dims,
                        const Tensor& positions,
                        const std::optional<Tensor>& cos_t,
                        const std::optional<Tensor>& sin_t,
                        const Tensor& q_mult, Tensor& k_cache,
                        Tensor& v_cache, const Tensor& slot_mapping) {
    const int c = act_code(q, "q");
    check_f32(q_norm, "q_norm");
    check_f32(k_norm, "k_norm");
    check_f32(q_mult, "q_mult");
    check_i32(positions, "positions");
    check_i32(slot_mapping, "slot_mapping");
    TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && q.stride(2) == 1 &&
                k.stride(2) == 1 && k.scalar_type() == q.scalar_type() &&
                k.is_cuda());
    const long T = q.size(0);
    const int H = (int)q.size(1), D = (int)q.size(2), G = (int)k.size(1);
    TORCH_CHECK(k.size(0) == T && k.size(2) == D && q.stride(1) == D &&
                k.stride(1) == D);
    TORCH_CHECK(q_norm.numel() == D && k_norm.numel() == D &&
                q_mult.numel() == H);
    TORCH_CHECK(rope_dims >= 0 && rope_dims % 2 == 0 && rope_dims <= D);
    const float *cp = nullptr, *sp = nullptr;
    if (rope_dims > 0) {
        TORCH_CHECK(cos_t.has_value() && sin_t.has_value());
        check_f32(*cos_t, "cos");
        check_f32(*sin_t, "sin");
        TORCH_CHECK(cos_t->dim() == 2 && cos_t->size(1) == rope_dims / 2 &&
                    sin_t->sizes() == cos_t->sizes());
        cp = cos_t->data_ptr<float>();
        sp = sin_t->data_ptr<float>();
    }
    for (const Tensor* t : {&k_cache, &v_cache})
        TORCH_CHECK(t->is_cuda() && t->scalar_type() == q.scalar_type() &&
                    t->is_contiguous() && t->dim() == 4 && t->size(1) == G &&
                    t->size(3) == D && t->sizes() == k_cache.sizes());
    TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
    const int rc = launch_qk_norm_rope_store(
        q.data_ptr(), q.stride(0), H, k.data_ptr(), k.stride(0), G, D,
        q_norm.data_ptr<float>(), k_norm.data_ptr<float>(), (float)eps,
        (int)rope_dims, positions.data_ptr<int>(), cp, sp,
        q_mult.data_ptr<float>(), k_cache.data_ptr(), v_cache.data_ptr(),
        (int)k_cache.size(2), slot_mapping.data_ptr<int>(), T, c, stream());
    TORCH_CHECK(rc == 0, "qk_norm_rope_store: head dim must be <= 512");
}

void sink_attn(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache,
               const Tensor& block_table, const Tensor& positions,
               const Tensor& seq_idx, const Tensor& cu,
               const std::optional<Tensor>& sink, int64_t window, Tensor& out,
               double out_scale, int64_t max_qlen,
               const std::optional<Tensor>& head_gate) {
    const int c = act_code(q, "q");
    check_i32(block_table, "block_table");
    check_i32(positions, "positions");
    check_i32(seq_idx, "seq_idx");
    TORCH_CHECK(q.dim() == 3 && q.stride(2) == 1 && q.stride(1) == q.size(2));
    const int Tn = (int)q.size(0), H = (int)q.size(1), D = (int)q.size(2);
    TORCH_CHECK(k_cache.is_cuda() && k_cache.is_contiguous() &&
                k_cache.dim() == 4 && k_cache.size(3) == D &&
                k_cache.scalar_type() == q.scalar_type());
    const int G = (int)k_cache.size(1), bs = (int)k_cache.size(2);
    TORCH_CHECK(v_cache.is_cuda() && v_cache.is_contiguous() &&
                v_cache.dim() == 4 && v_cache.size(0) == k_cache.size(0) &&
                v_cache.size(1) == G && v_cache.size(2) == bs &&
                v_cache.scalar_type() == q.scalar_type());
    const int Dv = (int)v_cache.size(3);
    TORCH_CHECK(G >= 1 && H % G == 0 && window >= 0);
    TORCH_CHECK(block_table.dim() == 2 && positions.numel() == Tn &&
                seq_idx.numel() == Tn);
    check_slice(out, Tn, (long)H * Dv, q.scalar_type(), "out");
    const float* sk = nullptr;
    if (sink.has_value()) {
        check_f32(*sink, "sink");
        TORCH_CHECK(sink->numel() == H);
        sk = sink->data_ptr<float>();
    }
    check_i32(cu, "cu_seqlens");
    const void* hg = nullptr;
    long hg_tok = 0;
    if (head_gate.has_value()) {
        // raw gate, one number per (token, head), a column slice
        check_slice(*head_gate, Tn, H, q.scalar_type(), "head_gate");
        hg = head_gate->data_ptr();
        hg_tok = head_gate->stride(0);
    }
    // bf16 prompt portions with head size 64/128 run on the matrix cores
    // (the dense models' paged prefill kernel, with the weights as a bf16
    // pair, window-aware tile skipping, and the sink and head gate in its
    // epilogue); single rows in the same step ride along. fp32, other head
    // sizes and pure decode steps take the generic kernel below.
    if (c == 0 && max_qlen >= 16 && D == Dv && (D == 64 || D == 128)) {
        const long B = cu.numel() - 1;
        TORCH_CHECK(block_table.size(0) == B);
        Tensor last = cu.slice(0, 1, B + 1).to(torch::kLong) - 1;
        Tensor seq_lens =
            (positions.index_select(0, last.clamp_min(0)) + 1)
                .to(torch::kInt32);
        const int rc = launch_attn_prefill_paged_sink(
            (const unsigned short*)q.data_ptr(), q.stride(0),
            (const unsigned short*)k_cache.data_ptr(),
            (const unsigned short*)v_cache.data_ptr(), cu.data_ptr<int>(),
            block_table.data_ptr<int>(), seq_lens.data_ptr<int>(),
            (unsigned short*)out.data_ptr(), out.stride(0), (int)B, H, G, D,
            (int)block_table.size(1), bs, (int)max_qlen, sk,
            (float)out_scale, (int)window, (const unsigned short*)hg, hg_tok,
            stream());
        TORCH_CHECK(rc == 0, "sink_attn: matrix-core path refused a shape "
                             "its guard admitted");
        return;
    }
    // few rows (decode): split each row's keys over more waves, at least 64
    // keys per share of the longest context the tables can hold
    const long ctx = window > 0 ? window : block_table.size(1) * (long)bs;
    // a wave serves up to 4 query heads of one key group (mixers.hip)
    const long group = H / G;
    const long units = H / (group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1);
    long splits = 8192 / std::max<long>(1, (long)Tn * units);
    splits = std::min<long>({splits, 32, (ctx + 63) / 64});
    splits = std::max<long>(splits, 1);
    Tensor part_acc, part_ml;
    float *pa = nullptr, *pm = nullptr;
    if (splits > 1) {
        auto f32opt = q.options().dtype(torch::kFloat32);
        part_acc = torch::empty({splits, H, Tn, Dv}, f32opt);
        part_ml = torch::empty({splits, H, Tn, 2}, f32opt);
        pa = part_acc.data_ptr<float>();
        pm = part_ml.data_ptr<float>();
    }
    const int rc = launch_sink_attn(
        q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
        block_table.data_ptr<int>(), (int)block_table.size(1),
        positions.data_ptr<int>(), seq_idx.data_ptr<int>(), sk,
        out.data_ptr(), out.stride(0), (float)out_scale, pa, pm, (int)splits,
        Tn, H, G, D, Dv, bs, (int)window, c, hg, hg_tok, stream());
    TORCH_CHECK(rc == 0, "sink_attn: head sizes must be <= 256");
}

}  // namespace

void register_hybrid_ops(pybind11::module_& m) {
    m.def("scalar_rmsnorm", &scalar_rmsnorm, "RMS norm with one scalar gain");
    m.def("add_scalar_rmsnorm", &add_scalar_rmsnorm,
          "resid += unit(y)*g_post; out = unit(resid)*g_pre");
    m.def("gated_rmsnorm", &gated_rmsnorm, "unit(x) * w * sigmoid(gate)");
    m.def("clamped_glu", &clamped_glu, "clamped GLU activation");
    m.def("canon_conv", &canon_conv, "h + causal per-channel conv, carried state");
    m.def("latent_rope_store", &latent_rope_store,
          "latent norm + rotation + paged store; q rotation in place");
    m.def("latent_attn", &latent_attn,
          "windowed attention over the paged latent cache (absorbed form)",
          pybind11::arg("q_abs"), pybind11::arg("q_rot"),
          pybind11::arg("gate"), pybind11::arg("cache"),
          pybind11::arg("block_table"), pybind11::arg("positions"),
          pybind11::arg("seq_idx"), pybind11::arg("cu_seqlens"),
          pybind11::arg("window"), pybind11::arg("scale"),
          pybind11::arg("max_qlen"), pybind11::arg("sink") = std::nullopt);
    m.def("lightning_attn", &lightning_attn,
          "decayed linear attention with carried fp32 state");
    m.def("retention_attn", &retention_attn,
          "decayed linear attention on rotated q/k, carried fp32 state");
    m.def("add_rmsnorm_f32", &add_rmsnorm_f32,
          "resid(fp32) += y; out = unit(resid) * w");
    m.def("relu2", &relu2, "relu(x)^2 over column slices");
    m.def("short_conv", &short_conv,
          "causal per-channel conv (+silu) with carried state -> fp32");
    m.def("delta_gates", &delta_gates,
          "unit q/k in place, beta and decay of a delta-rule step");
    m.def("delta_rule", &delta_rule,
          "gated delta rule with carried fp32 state");
    m.def("head_gated_norm", &head_gated_norm,
          "per-head unit(o) * w * act(gate) into a column slice");
    m.def("qk_norm_rope_store", &qk_norm_rope_store,
          "q/k head norm + rotation; keys and raw keys to the pages");
    m.def("sink_attn", &sink_attn,
          "paged causal GQA softmax attention with a sink logit",
          pybind11::arg("q"), pybind11::arg("k_cache"),
          pybind11::arg("v_cache"), pybind11::arg("block_table"),
          pybind11::arg("positions"), pybind11::arg("seq_idx"),
          pybind11::arg("cu_seqlens"), pybind11::arg("sink"),
          pybind11::arg("window"), pybind11::arg("out"),
          pybind11::arg("out_scale"), pybind11::arg("max_qlen"),
          pybind11::arg("head_gate") = std::nullopt);
}
