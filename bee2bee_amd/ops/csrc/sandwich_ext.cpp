// Torch bindings for the weighted-sandwich stack kernels (sandwich.hip and
// the head-mixing attention in mixers.hip / attn_prefill.hip). Shapes,
// strides and dtypes are validated here so the kernels index without
// checks. Activations are bf16 or fp32; residual, norm weights, the
// head-mixing matrix and all partial sums are fp32. All entry points are
// hipGraph-capture safe (no sync, no host reads).
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <optional>
#include <vector>

using torch::Tensor;

extern "C" {
int launch_add_group_rmsnorm(float*, const void*, const float*, const float*,
                             const float*, void*, long, int, int, float, int,
                             int, hipStream_t);
int launch_rope_unit_store(void*, long, int, const void*, long, const void*,
                           long, int, int, int, float, int, const int*,
                           const float*, const float*, float, void*, void*,
                           int, const int*, long, int, hipStream_t);
void launch_polynorm(const void*, const float*, void*, long, int, float, int,
                     hipStream_t);
void launch_silu_glu(const void*, void*, long, long, int, hipStream_t);
int launch_talk_attn(const void*, long, const void*, const void*, const int*,
                     int, const int*, const int*, float*, float*, int, int,
                     int, int, int, int, int, int, int, hipStream_t);
int launch_talk_attn_scored(const void*, long, const void*, const void*,
                            const int*, int, const int*, const int*,
                            const float*, const void*, long, void*, long,
                            float*, long, float*, float*, int, int, int, int,
                            int, int, int, int, int, hipStream_t);
int launch_talk_mix(const float*, const float*, const float*, const void*,
                    long, void*, long, int, int, int, int, int, int,
                    hipStream_t);
int launch_attn_prefill_paged_cross(const unsigned short*, long,
                                    const unsigned short*,
                                    const unsigned short*, const int*,
                                    const int*, const int*, float*, int, int,
                                    int, int, int, int, int, int,
                                    hipStream_t);
}

namespace {

inline hipStream_t stream() {
    return at::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
}

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

void check_slice(const Tensor& t, long T, long n, at::ScalarType dt,
                 const char* name) {
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == dt && t.dim() == 2 &&
                    t.size(0) == T && t.size(1) == n &&
                    (n == 1 || t.stride(1) == 1),
                name, ": expected a [", T, ", ", n, "] column slice");
}

std::optional<Tensor> add_group_rmsnorm(
    Tensor& resid, const std::optional<Tensor>& y,
    const std::optional<Tensor>& w_post, const std::optional<Tensor>& step,
    const std::optional<Tensor>& w_pre, int64_t groups, double eps,
    at::ScalarType out_dtype) {
    check_f32(resid, "resid");
    TORCH_CHECK(resid.dim() == 2);
    const long T = resid.size(0);
    const int W = (int)resid.size(1);
    const void* yp = nullptr;
    const float *wpost = nullptr, *sp = nullptr, *wpre = nullptr;
    int yc = 1;
    if (y.has_value()) {
        TORCH_CHECK(y->sizes() == resid.sizes() && y->is_contiguous() &&
                    w_post.has_value());
        yc = act_code(*y, "y");
        yp = y->data_ptr();
        check_f32(*w_post, "w_post");
        TORCH_CHECK(w_post->numel() == W);
        wpost = w_post->data_ptr<float>();
    }
    if (step.has_value()) {
        check_f32(*step, "step");
        TORCH_CHECK(step->numel() == W);
        sp = step->data_ptr<float>();
    }
    const int oc = act_code(out_dtype, "out_dtype");
    std::optional<Tensor> out;
    void* op = nullptr;
    if (w_pre.has_value()) {
        check_f32(*w_pre, "w_pre");
        TORCH_CHECK(w_pre->numel() == W);
        wpre = w_pre->data_ptr<float>();
        out = torch::empty(resid.sizes(), resid.options().dtype(out_dtype));
        op = out->data_ptr();
    }
    if (!yp && !sp && !op) return out;
    // two fp32 rows in LDS when y is given
    TORCH_CHECK((size_t)W * 4 * (yp ? 2 : 1) <= 60 * 1024,
                "add_group_rmsnorm: row too wide for the LDS-resident kernel");
    const int rc = launch_add_group_rmsnorm(
        resid.data_ptr<float>(), yp, wpost, sp, wpre, op, T, W, (int)groups,
        (float)eps, yc, oc, stream());
    TORCH_CHECK(rc == 0, "add_group_rmsnorm: groups must divide the width "
                         "and be <= 64");
    return out;
}

void rope_unit_store(Tensor& q, const Tensor& k, const Tensor& v, double eps,
                     int64_t rope_dims, const Tensor& positions,
                     const std::optional<Tensor>& cos_t,
                     const std::optional<Tensor>& sin_t, double q_mult,
                     Tensor& k_cache, Tensor& v_cache,
                     const Tensor& slot_mapping) {
    const int c = act_code(q, "q");
    check_i32(positions, "positions");
    check_i32(slot_mapping, "slot_mapping");
    TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3 &&
                q.stride(2) == 1 && k.stride(2) == 1 && v.stride(2) == 1 &&
                k.scalar_type() == q.scalar_type() &&
                v.scalar_type() == q.scalar_type() && k.is_cuda() &&
                v.is_cuda());
    const long T = q.size(0);
    const int H = (int)q.size(1), D = (int)q.size(2), G = (int)k.size(1);
    const int Dv = (int)v.size(2);
    TORCH_CHECK(k.size(0) == T && v.size(0) == T && k.size(2) == D &&
                v.size(1) == G && q.stride(1) == D && k.stride(1) == D &&
                v.stride(1) == Dv);
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
    TORCH_CHECK(k_cache.is_cuda() && k_cache.is_contiguous() &&
                k_cache.dim() == 4 && k_cache.size(1) == G &&
                k_cache.size(3) == D &&
                k_cache.scalar_type() == q.scalar_type());
    TORCH_CHECK(v_cache.is_cuda() && v_cache.is_contiguous() &&
                v_cache.dim() == 4 && v_cache.size(0) == k_cache.size(0) &&
                v_cache.size(1) == G && v_cache.size(2) == k_cache.size(2) &&
                v_cache.size(3) == Dv &&
                v_cache.scalar_type() == q.scalar_type());
    TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
    const int rc = launch_rope_unit_store(
        q.data_ptr(), q.stride(0), H, k.data_ptr(), k.stride(0), v.data_ptr(),
        v.stride(0), G, D, Dv, (float)eps, (int)rope_dims,
        positions.data_ptr<int>(), cp, sp, (float)q_mult, k_cache.data_ptr(),
        v_cache.data_ptr(), (int)k_cache.size(2),
        slot_mapping.data_ptr<int>(), T, c, stream());
    TORCH_CHECK(rc == 0, "rope_unit_store: head dim must be <= 512");
}

Tensor polynorm(const Tensor& z, const Tensor& coef, double eps,
                at::ScalarType out_dtype) {
    const int c = act_code(z, "z");
    check_f32(coef, "coef");
    TORCH_CHECK(z.dim() == 2 && z.is_contiguous() && coef.numel() == 4 &&
                out_dtype == z.scalar_type());
    Tensor out = torch::empty_like(z);
    launch_polynorm(z.data_ptr(), coef.data_ptr<float>(), out.data_ptr(),
                    z.size(0), (int)z.size(1), (float)eps, c, stream());
    return out;
}

Tensor silu_glu(const Tensor& gu) {
    const int c = act_code(gu, "gate_up");
    TORCH_CHECK(gu.is_contiguous() && gu.size(-1) % 2 == 0);
    const long I = gu.size(-1) / 2;
    const long rows = gu.numel() / (2 * I);
    auto shape = gu.sizes().vec();
    shape.back() = I;
    Tensor y = torch::empty(shape, gu.options());
    launch_silu_glu(gu.data_ptr(), y.data_ptr(), rows, I, c, stream());
    return y;
}

void talk_attn(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache,
               const Tensor& block_table, const Tensor& positions,
               const Tensor& seq_idx, const Tensor& cu, const Tensor& talk,
               const Tensor& gate, int64_t window, Tensor& out,
               int64_t max_qlen, int64_t path) {
    // path: 0 = choose by dtype, head size and step shape; 1 = scores
    // written once, heads mixed before the values; 2 = every head's weights
    // against every value head, mixed afterwards (generic kernel)
    const int c = act_code(q, "q");
    check_i32(block_table, "block_table");
    check_i32(positions, "positions");
    check_i32(seq_idx, "seq_idx");
    check_i32(cu, "cu_seqlens");
    check_f32(talk, "talk");
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
    TORCH_CHECK(talk.dim() == 2 && talk.size(0) == H && talk.size(1) == H);
    TORCH_CHECK(block_table.dim() == 2 && positions.numel() == Tn &&
                seq_idx.numel() == Tn);
    check_slice(out, Tn, (long)H * Dv, q.scalar_type(), "out");
    check_slice(gate, Tn, (long)H * Dv, q.scalar_type(), "gate");
    if (Tn == 0) return;
    auto f32opt = q.options().dtype(torch::kFloat32);
    // bf16 prompt portions with head size 64/128 run on the matrix cores:
    // the paged prefill kernel applies every query head's weights (a bf16
    // hi+lo pair) to the values of all key/value heads; single rows of the
    // same step ride along. fp32, other head sizes and pure decode steps
    // take the generic kernel below.
    if (path == 0 && c == 0 && max_qlen >= 16 && D == Dv &&
        (D == 64 || D == 128)) {
        const long B = cu.numel() - 1;
        TORCH_CHECK(block_table.size(0) == B);
        Tensor last = cu.slice(0, 1, B + 1).to(torch::kLong) - 1;
        Tensor seq_lens =
            (positions.index_select(0, last.clamp_min(0)) + 1)
                .to(torch::kInt32);
        Tensor part = torch::empty({1, Tn, G, H, Dv}, f32opt);
        int rc = launch_attn_prefill_paged_cross(
            (const unsigned short*)q.data_ptr(), q.stride(0),
            (const unsigned short*)k_cache.data_ptr(),
            (const unsigned short*)v_cache.data_ptr(), cu.data_ptr<int>(),
            block_table.data_ptr<int>(), seq_lens.data_ptr<int>(),
            part.data_ptr<float>(), (int)B, H, G, D,
            (int)block_table.size(1), bs, (int)max_qlen, (int)window,
            stream());
        TORCH_CHECK(rc == 0, "talk_attn: matrix-core path refused a shape "
                             "its guard admitted");
        rc = launch_talk_mix(part.data_ptr<float>(), nullptr,
                             talk.data_ptr<float>(), gate.data_ptr(),
                             gate.stride(0), out.data_ptr(), out.stride(0), 1,
                             Tn, H, G, Dv, c, stream());
        TORCH_CHECK(rc == 0, "talk_attn: heads x value size too large for "
                             "the mixing kernel");
        return;
    }
    // few rows (decode): split each row's keys over more waves, at least 64
    // keys per share of the longest context the tables can hold
    const long cap = block_table.size(1) * (long)bs;
    const long ctx = window > 0 ? std::min<long>(window, cap) : cap;
    const long group = H / G;
    const long units = H / (group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1);
    // Steps whose score matrix [Tn, H, ctx] is small (decode rows, short
    // portions, windows): scores are written once and the heads are mixed
    // before the values are read, so each value row is read once per key
    // group. Larger fp32 / odd-size prompt steps apply every head's
    // weights to every value head and mix afterwards (below).
    if (path == 1 || (path == 0 && (long)Tn * H * ctx * 4 <= (256L << 20))) {
        long splits = 8192 / std::max<long>(1, (long)Tn * units);
        splits = std::min<long>({splits, 32, (ctx + 63) / 64});
        splits = std::max<long>(splits, 1);
        Tensor scores = torch::empty({Tn, H, ctx}, f32opt);
        Tensor part_ml = torch::empty({splits, Tn, H, 2}, f32opt);
        Tensor part_o;
        float* po = nullptr;
        if (splits > 1) {
            part_o = torch::empty({splits, Tn, H, Dv}, f32opt);
            po = part_o.data_ptr<float>();
        }
        const int rc = launch_talk_attn_scored(
            q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
            block_table.data_ptr<int>(), (int)block_table.size(1),
            positions.data_ptr<int>(), seq_idx.data_ptr<int>(),
            talk.data_ptr<float>(), gate.data_ptr(), gate.stride(0),
            out.data_ptr(), out.stride(0), scores.data_ptr<float>(), ctx,
            part_ml.data_ptr<float>(), po, (int)splits, Tn, H, G, D, Dv, bs,
            (int)window, c, stream());
        TORCH_CHECK(rc == 0, "talk_attn: head sizes must be <= 256");
        return;
    }
    const long nv = G >= 4 ? 4 : G >= 2 ? 2 : 1;
    const long waves = (long)Tn * units * ((G + nv - 1) / nv);
    long splits = 8192 / std::max<long>(1, waves);
    splits = std::min<long>({splits, 32, (ctx + 63) / 64});
    splits = std::max<long>(splits, 1);
    Tensor part_acc = torch::empty({splits, Tn, G, H, Dv}, f32opt);
    Tensor part_ml = torch::empty({splits, Tn, H, 2}, f32opt);
    int rc = launch_talk_attn(
        q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
        block_table.data_ptr<int>(), (int)block_table.size(1),
        positions.data_ptr<int>(), seq_idx.data_ptr<int>(),
        part_acc.data_ptr<float>(), part_ml.data_ptr<float>(), (int)splits,
        Tn, H, G, D, Dv, bs, (int)window, c, stream());
    TORCH_CHECK(rc == 0, "talk_attn: head sizes must be <= 256");
    rc = launch_talk_mix(part_acc.data_ptr<float>(),
                         part_ml.data_ptr<float>(), talk.data_ptr<float>(),
                         gate.data_ptr(), gate.stride(0), out.data_ptr(),
                         out.stride(0), (int)splits, Tn, H, G, Dv, c,
                         stream());
    TORCH_CHECK(rc == 0, "talk_attn: heads x value size too large for the "
                         "mixing kernel");
}

}  // namespace

void register_sandwich_ops(pybind11::module_& m) {
    m.def("add_group_rmsnorm", &add_group_rmsnorm,
          "resid += gnorm(y)*w_post [+ step]; out = gnorm(resid)*w_pre");
    m.def("rope_unit_store", &rope_unit_store,
          "rotate, unit-norm q/k; keys and values to the pages");
    m.def("polynorm", &polynorm, "a unit(z) + b unit(z^2) + c unit(z^3) + e");
    m.def("silu_glu", &silu_glu, "silu(gate) * up");
    m.def("talk_attn", &talk_attn,
          "paged windowed GQA attention with head-mixed softmax weights "
          "and a sigmoid output gate");
}
