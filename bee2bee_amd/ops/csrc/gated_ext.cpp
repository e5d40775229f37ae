// Torch bindings for the gated parallel-form kernels (gated.hip) and the
// score-mixing attention (mixers.hip). Shapes, strides and dtypes are
// validated here so the kernels index without checks. Activations are bf16
// or fp32; residual, norm weights, rotation tables and recurrent state are
// fp32. All entry points are hipGraph-capture safe (no sync, no host reads).
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <optional>
#include <vector>

using torch::Tensor;

extern "C" {
void launch_gated_add_rmsnorm(float*, const void*, const void*, long,
                              const void*, const void*, long, const float*,
                              const float*, void*, long, int, float, int, int,
                              int, hipStream_t);
void launch_pair_rmsnorm_mean(const void*, const float*, const void*,
                              const float*, void*, long, int, float, int, int,
                              hipStream_t);
void launch_slice_rmsnorm(const void*, long, const float*, void*, long, int,
                          float, int, hipStream_t);
void launch_gelu_erf(const void*, void*, long, int, hipStream_t);
int launch_rope_store(const void*, long, void*, long, int, const void*, long,
                      const void*, long, int, int, int, int, int, const int*,
                      const float*, const float*, float, void*, void*, int,
                      const int*, long, int, int, hipStream_t);
int min_gru_segment_tokens();
void launch_min_gru(const void*, long, const void*, long, const void*, long,
                    float*, const int*, const int*, const int*, void*, long,
                    float*, float*, int, int, int, int, hipStream_t);
int launch_mixed_score_attn(const void*, long, const void*, const void*,
                            const int*, int, const int*, const int*, float,
                            const float*, const float*, const void*, long,
                            void*, long, float*, long, float*, float*, float*,
                            int, int, int, int, int, int, int, int, int,
                            hipStream_t);
int launch_group_topk_gate(const float*, float*, int*, long, int, int, int,
                           int, int, int, hipStream_t);
int launch_attn_prefill_paged_mixed(
    const unsigned short*, long, const unsigned short*, const unsigned short*,
    const int*, const int*, const int*, unsigned short*, long, int, int, int,
    int, int, int, int, int, float*, long, float, const float*, const float*,
    int, const unsigned short*, long, hipStream_t);
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

// a [T, n] view with unit column stride (a column slice of a wider buffer)
void check_slice(const Tensor& t, long T, long n, at::ScalarType dt,
                 const char* name) {
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == dt && t.dim() == 2 &&
                    t.size(0) == T && t.size(1) == n &&
                    (n == 1 || t.stride(1) == 1),
                name, ": expected a [", T, ", ", n, "] column slice");
}

// rows, row stride and base address allow 4-element accesses
bool aligned4(const Tensor& t) {
    return t.size(-1) % 4 == 0 && (t.dim() < 2 || t.stride(0) % 4 == 0) &&
           reinterpret_cast<uintptr_t>(t.data_ptr()) %
                   (4 * t.element_size()) == 0;
}

std::optional<Tensor> gated_add_rmsnorm(
    Tensor& resid, const std::optional<Tensor>& y1,
    const std::optional<Tensor>& g1, const std::optional<Tensor>& y2,
    const std::optional<Tensor>& g2, const std::optional<Tensor>& extra,
    const std::optional<Tensor>& w, double eps, at::ScalarType out_dtype) {
    check_f32(resid, "resid");
    TORCH_CHECK(resid.dim() == 2);
    const long T = resid.size(0);
    const int W = (int)resid.size(1);
    TORCH_CHECK(W * sizeof(float) <= 64 * 1024, "row too wide");
    const int oc = act_code(out_dtype, "out_dtype");
    int yc = oc;
    bool vec = aligned4(resid);
    const void *y1p = nullptr, *g1p = nullptr, *y2p = nullptr, *g2p = nullptr;
    long gs1 = 0, gs2 = 0;
    TORCH_CHECK(y1.has_value() || !y2.has_value(),
                "a second sublayer needs the first");
    if (y1.has_value()) {
        yc = act_code(*y1, "y1");
        TORCH_CHECK(g1.has_value());
        TORCH_CHECK(y1->is_contiguous() && y1->sizes() == resid.sizes());
        check_slice(*g1, T, W, y1->scalar_type(), "g1");
        y1p = y1->data_ptr();
        g1p = g1->data_ptr();
        gs1 = g1->stride(0);
        vec = vec && aligned4(*y1) && aligned4(*g1);
    }
    if (y2.has_value()) {
        TORCH_CHECK(g2.has_value());
        TORCH_CHECK(y2->is_cuda() && y2->is_contiguous() &&
                    y2->sizes() == resid.sizes() &&
                    y2->scalar_type() == y1->scalar_type());
        check_slice(*g2, T, W, y1->scalar_type(), "g2");
        y2p = y2->data_ptr();
        g2p = g2->data_ptr();
        gs2 = g2->stride(0);
        vec = vec && aligned4(*y2) && aligned4(*g2);
    }
    const float* ep = nullptr;
    if (extra.has_value()) {
        check_f32(*extra, "extra");
        TORCH_CHECK(extra->sizes() == resid.sizes());
        ep = extra->data_ptr<float>();
        vec = vec && aligned4(*extra);
    }
    std::optional<Tensor> out;
    void* op = nullptr;
    const float* wp = nullptr;
    if (w.has_value()) {
        check_f32(*w, "w");
        TORCH_CHECK(w->numel() == W);
        wp = w->data_ptr<float>();
        out = torch::empty(resid.sizes(), resid.options().dtype(out_dtype));
        op = out->data_ptr();
        vec = vec && aligned4(*w);
    }
    launch_gated_add_rmsnorm(resid.data_ptr<float>(), y1p, g1p, gs1, y2p, g2p,
                             gs2, ep, wp, op, T, W, (float)eps, yc, oc,
                             vec ? 1 : 0, stream());
    return out;
}

Tensor pair_rmsnorm_mean(const Tensor& a, const Tensor& wa, const Tensor& b,
                         const Tensor& wb, double eps,
                         at::ScalarType out_dtype) {
    const int c = act_code(a, "a");
    TORCH_CHECK(out_dtype == a.scalar_type(),
                "inputs and output share the activation dtype");
    check_f32(wa, "wa");
    check_f32(wb, "wb");
    TORCH_CHECK(a.dim() == 2 && a.is_contiguous() && b.is_cuda() &&
                b.is_contiguous() && b.sizes() == a.sizes() &&
                b.scalar_type() == a.scalar_type());
    const int W = (int)a.size(1);
    TORCH_CHECK(wa.numel() == W && wb.numel() == W);
    TORCH_CHECK(2 * W * sizeof(float) <= 64 * 1024, "row too wide");
    Tensor out = torch::empty_like(a);
    const bool vec = aligned4(a) && aligned4(b) && aligned4(out) &&
                     aligned4(wa) && aligned4(wb);
    launch_pair_rmsnorm_mean(a.data_ptr(), wa.data_ptr<float>(), b.data_ptr(),
                             wb.data_ptr<float>(), out.data_ptr(), a.size(0),
                             W, (float)eps, c, vec ? 1 : 0, stream());
    return out;
}

Tensor slice_rmsnorm(const Tensor& x, const Tensor& w, double eps) {
    const int c = act_code(x, "x");
    check_f32(w, "w");
    TORCH_CHECK(x.dim() == 2);
    const long T = x.size(0);
    const int N = (int)x.size(1);
    check_slice(x, T, N, x.scalar_type(), "x");
    TORCH_CHECK(w.numel() == N);
    Tensor out = torch::empty({T, (long)N}, x.options());
    launch_slice_rmsnorm(x.data_ptr(), x.stride(0), w.data_ptr<float>(),
                         out.data_ptr(), T, N, (float)eps, c, stream());
    return out;
}

Tensor gelu_erf(const Tensor& x) {
    const int c = act_code(x, "x");
    TORCH_CHECK(x.is_contiguous());
    Tensor y = torch::empty_like(x);
    launch_gelu_erf(x.data_ptr(), y.data_ptr(), x.numel(), c, stream());
    return y;
}

void rope_store(const Tensor& q, const Tensor& k, const Tensor& v,
                Tensor& q_out, int64_t rope_dims, bool interleaved,
                const Tensor& positions, const std::optional<Tensor>& cos_t,
                const std::optional<Tensor>& sin_t, double q_mult,
                Tensor& k_cache, Tensor& v_cache,
                const Tensor& slot_mapping) {
    const int c = act_code(q_out, "q_out");
    const int in_f32 = act_code(q, "q");
    TORCH_CHECK(in_f32 || !c, "fp32 pages need fp32 inputs");
    check_i32(positions, "positions");
    check_i32(slot_mapping, "slot_mapping");
    auto head_view = [&](const Tensor& t, const char* name) {
        TORCH_CHECK(t.is_cuda() && t.dim() == 3 && t.stride(2) == 1 &&
                        t.stride(1) == t.size(2),
                    name, ": expected [T, heads, dim] rows of whole heads");
    };
    head_view(q, "q");
    head_view(k, "k");
    head_view(v, "v");
    head_view(q_out, "q_out");
    TORCH_CHECK(k.scalar_type() == q.scalar_type() &&
                v.scalar_type() == q.scalar_type());
    const long T = q.size(0);
    const int H = (int)q.size(1), D = (int)q.size(2);
    const int G = (int)k.size(1), Dv = (int)v.size(2);
    TORCH_CHECK(q_out.sizes() == q.sizes());
    TORCH_CHECK(k.size(0) == T && v.size(0) == T && k.size(2) == D &&
                v.size(1) == G);
    TORCH_CHECK(k_cache.is_cuda() && k_cache.is_contiguous() &&
                k_cache.dim() == 4 && k_cache.size(1) == G &&
                k_cache.size(3) == D &&
                k_cache.scalar_type() == q_out.scalar_type());
    const int bs = (int)k_cache.size(2);
    TORCH_CHECK(v_cache.is_cuda() && v_cache.is_contiguous() &&
                v_cache.dim() == 4 && v_cache.size(0) == k_cache.size(0) &&
                v_cache.size(1) == G && v_cache.size(2) == bs &&
                v_cache.size(3) == Dv &&
                v_cache.scalar_type() == q_out.scalar_type());
    TORCH_CHECK(rope_dims >= 0 && rope_dims <= D && rope_dims % 2 == 0);
    TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
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
    const int rc = launch_rope_store(
        q.data_ptr(), q.stride(0), q_out.data_ptr(), q_out.stride(0), H,
        k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), G, D, Dv,
        (int)rope_dims, interleaved ? 1 : 0, positions.data_ptr<int>(), cp,
        sp, (float)q_mult, k_cache.data_ptr(), v_cache.data_ptr(), bs,
        slot_mapping.data_ptr<int>(), T, in_f32, c, stream());
    TORCH_CHECK(rc == 0, "rope_store: head dim must be <= 512");
}

void min_gru(const Tensor& z, const Tensor& x, const Tensor& g, Tensor& state,
             const Tensor& state_slots, const Tensor& cu,
             const Tensor& positions, Tensor& out, int64_t max_qlen) {
    const int c = act_code(z, "z");
    check_f32(state, "state");
    check_i32(state_slots, "state_slots");
    check_i32(cu, "cu_seqlens");
    check_i32(positions, "positions");
    TORCH_CHECK(z.dim() == 2);
    const long T = z.size(0);
    const int N = (int)z.size(1);
    check_slice(z, T, N, z.scalar_type(), "z");
    check_slice(x, T, N, z.scalar_type(), "x");
    check_slice(g, T, N, z.scalar_type(), "g");
    check_slice(out, T, N, z.scalar_type(), "out");
    const int B = (int)cu.numel() - 1;
    TORCH_CHECK(state.dim() == 2 && state.size(1) == N &&
                state_slots.numel() == B && positions.numel() == T);
    // long portions: segments in parallel + a scan over their (decay, end
    // state) pairs; the bound on the segment count needs no host read
    const int seg = min_gru_segment_tokens();
    int n_seg = 0;
    Tensor ws;
    float *wp = nullptr, *wl = nullptr;
    if (max_qlen > 2 * seg) {
        n_seg = (int)(T / seg) + B;
        ws = torch::empty({2, (long)n_seg, (long)N},
                          state.options().dtype(torch::kFloat32));
        wp = ws.data_ptr<float>();
        wl = wp + (long)n_seg * N;
    }
    launch_min_gru(z.data_ptr(), z.stride(0), x.data_ptr(), x.stride(0),
                   g.data_ptr(), g.stride(0), state.data_ptr<float>(),
                   state_slots.data_ptr<int>(), cu.data_ptr<int>(),
                   positions.data_ptr<int>(), out.data_ptr(), out.stride(0),
                   wp, wl, n_seg, B, N, c, stream());
}

// Grouped-query attention whose capped scores are mixed across heads before
// the softmax. The scores of a block of rows are written once ([rows, H,
// ctx] fp32, at most ~256 MB per block; longer steps run block by block).
// bf16 prompt portions (max_qlen >= 16) with head size 64/128 run on the
// matrix cores: tile scores, the mix, then softmax and P V from the mixed
// tiles; fp32, other head sizes and decode steps take the wave-per-row
// kernels.
void mixed_score_attn(const Tensor& q, const Tensor& k_cache,
                      const Tensor& v_cache, const Tensor& block_table,
                      const Tensor& positions, const Tensor& seq_idx,
                      const Tensor& cu, double softcap, const Tensor& mix,
                      const std::optional<Tensor>& sink,
                      const std::optional<Tensor>& head_gate, int64_t window,
                      Tensor& out, int64_t max_qlen) {
    const int c = act_code(q, "q");
    check_i32(block_table, "block_table");
    check_i32(positions, "positions");
    check_i32(seq_idx, "seq_idx");
    check_f32(mix, "mix");
    TORCH_CHECK(q.dim() == 3 && q.stride(2) == 1 && q.stride(1) == q.size(2));
    const long Tn = q.size(0);
    const int H = (int)q.size(1), D = (int)q.size(2);
    TORCH_CHECK(k_cache.is_cuda() && k_cache.is_contiguous() &&
                k_cache.dim() == 4 && k_cache.size(3) == D &&
                k_cache.scalar_type() == q.scalar_type());
    const int G = (int)k_cache.size(1), bs = (int)k_cache.size(2);
    TORCH_CHECK(v_cache.is_cuda() && v_cache.is_contiguous() &&
                v_cache.dim() == 4 && v_cache.size(0) == k_cache.size(0) &&
                v_cache.size(1) == G && v_cache.size(2) == bs &&
                v_cache.scalar_type() == q.scalar_type());
    const int Dv = (int)v_cache.size(3);
    TORCH_CHECK(G >= 1 && H % G == 0 && window >= 0 && softcap >= 0);
    TORCH_CHECK(mix.dim() == 2 && mix.size(0) == H && mix.size(1) == H);
    TORCH_CHECK(block_table.dim() == 2 && positions.numel() == Tn &&
                seq_idx.numel() == Tn);
    check_slice(out, Tn, (long)H * Dv, q.scalar_type(), "out");
    const float* sk = nullptr;
    if (sink.has_value()) {
        check_f32(*sink, "sink");
        TORCH_CHECK(sink->numel() == H);
        sk = sink->data_ptr<float>();
    }
    const char* hg = nullptr;
    long hg_tok = 0;
    if (head_gate.has_value()) {
        check_slice(*head_gate, Tn, H, q.scalar_type(), "head_gate");
        hg = (const char*)head_gate->data_ptr();
        hg_tok = head_gate->stride(0);
    }
    if (Tn == 0) return;
    check_i32(cu, "cu_seqlens");
    // the most keys a row can see, in whole 64-key tiles
    const long reach = block_table.size(1) * (long)bs;
    auto f32opt = q.options().dtype(torch::kFloat32);
    if (c == 0 && max_qlen >= 16 && D == Dv && (D == 64 || D == 128) &&
        (size_t)H * H * 4 + (size_t)H * 1024 <= 64 * 1024) {
        const long B = cu.numel() - 1;
        TORCH_CHECK(block_table.size(0) == B);
        Tensor last = cu.slice(0, 1, B + 1).to(torch::kLong) - 1;
        Tensor seq_lens =
            (positions.index_select(0, last.clamp_min(0)) + 1)
                .to(torch::kInt32);
        // a 64-query tile visits at most window + 126 keys, in 64-key tiles
        long tctx = window > 0 ? std::min<long>(window + 128, reach + 64)
                               : reach + 64;
        tctx = (tctx + 63) / 64 * 64;
        const long tiles = (max_qlen + 63) / 64;
        // tiles per launch: a score buffer of at most ~256 MB
        const long per =
            std::max<long>(1, (64L << 20) / (B * 64 * H * tctx));
        const long nt = std::min<long>(tiles, per);
        Tensor buf = torch::empty({B, nt * 64, (long)H, tctx}, f32opt);
        for (long t0 = 0; t0 < tiles; t0 += nt) {
            const int rc = launch_attn_prefill_paged_mixed(
                (const unsigned short*)q.data_ptr(), q.stride(0),
                (const unsigned short*)k_cache.data_ptr(),
                (const unsigned short*)v_cache.data_ptr(),
                cu.data_ptr<int>(), block_table.data_ptr<int>(),
                seq_lens.data_ptr<int>(), (unsigned short*)out.data_ptr(),
                out.stride(0), (int)B, H, G, D, (int)block_table.size(1), bs,
                (int)t0, (int)std::min<long>(nt, tiles - t0),
                buf.data_ptr<float>(), tctx, (float)softcap,
                mix.data_ptr<float>(), sk, (int)window,
                (const unsigned short*)hg, hg_tok, stream());
            TORCH_CHECK(rc == 0, "mixed_score_attn: matrix-core path refused "
                                 "a shape its guard admitted");
        }
        return;
    }
    long ctx = window > 0 ? std::min<long>(window, reach) : reach;
    ctx = (ctx + 63) / 64 * 64;
    const long block_rows = std::max<long>(
        1, std::min<long>(Tn, (64L << 20) / std::max<long>(1, H * ctx)));
    const long group = H / G;
    const long units = H / (group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1);
    long splits = 8192 / std::max<long>(1, block_rows * units);
    splits = std::min<long>({splits, 32, (ctx + 63) / 64});
    splits = std::max<long>(splits, 1);
    Tensor scores = torch::empty({block_rows, (long)H, ctx}, f32opt);
    Tensor scratch = torch::empty({splits, block_rows, (long)H, 2}, f32opt);
    Tensor part_acc, part_ml;
    float *pa = nullptr, *pm = nullptr;
    if (splits > 1) {
        part_acc = torch::empty({splits, (long)H, block_rows, (long)Dv},
                                f32opt);
        part_ml = torch::empty({splits, (long)H, block_rows, 2}, f32opt);
        pa = part_acc.data_ptr<float>();
        pm = part_ml.data_ptr<float>();
    }
    const long esz = q.element_size();
    for (long t0 = 0; t0 < Tn; t0 += block_rows) {
        const int rows = (int)std::min<long>(block_rows, Tn - t0);
        const int rc = launch_mixed_score_attn(
            (const char*)q.data_ptr() + t0 * q.stride(0) * esz, q.stride(0),
            k_cache.data_ptr(), v_cache.data_ptr(),
            block_table.data_ptr<int>(), (int)block_table.size(1),
            positions.data_ptr<int>() + t0, seq_idx.data_ptr<int>() + t0,
            (float)softcap, mix.data_ptr<float>(), sk,
            hg ? hg + t0 * hg_tok * esz : nullptr, hg_tok,
            (char*)out.data_ptr() + t0 * out.stride(0) * esz, out.stride(0),
            scores.data_ptr<float>(), ctx, scratch.data_ptr<float>(), pa, pm,
            (int)splits, rows, H, G, D, Dv, bs, (int)window, c, stream());
        TORCH_CHECK(rc == 0, "mixed_score_attn: head sizes must be <= 256");
    }
}

std::vector<Tensor> group_topk_gate(const Tensor& logits, int64_t top_k,
                                    int64_t n_groups, int64_t keep,
                                    bool sigmoid, int64_t group_top) {
    check_f32(logits, "logits");
    TORCH_CHECK(logits.dim() == 2);
    const long T = logits.size(0);
    const int E = (int)logits.size(1);
    TORCH_CHECK(n_groups >= 1 && E % n_groups == 0 && keep >= 1 &&
                keep <= n_groups && top_k >= 1 &&
                top_k <= keep * (E / n_groups),
                "experts must split into equal groups and the kept groups "
                "must hold top_k experts");
    Tensor w = torch::empty({T, top_k}, logits.options());
    Tensor idx = torch::empty({T, top_k},
                              logits.options().dtype(torch::kInt32));
    const int rc = launch_group_topk_gate(
        logits.data_ptr<float>(), w.data_ptr<float>(), idx.data_ptr<int>(), T,
        E, (int)top_k, (int)n_groups, (int)keep, (int)group_top,
        sigmoid ? 1 : 0, stream());
    TORCH_CHECK(rc == 0, "group_topk_gate: too many experts for one "
                         "workgroup's LDS");
    return {w, idx};
}

}  // namespace

void register_gated_ops(pybind11::module_& m) {
    m.def("group_topk_gate", &group_topk_gate,
          "group-limited expert choice on sigmoid or softmax scores");
    m.def("gated_add_rmsnorm", &gated_add_rmsnorm,
          "resid += sigmoid(g1) y1 [+ sigmoid(g2) y2] [+ extra]; "
          "out = unit(resid) * w");
    m.def("pair_rmsnorm_mean", &pair_rmsnorm_mean,
          "(unit(a) * wa + unit(b) * wb) / 2");
    m.def("slice_rmsnorm", &slice_rmsnorm, "unit(x) * w on a column slice");
    m.def("gelu_erf", &gelu_erf, "exact gelu");
    m.def("rope_store", &rope_store,
          "rotate q/k (either pair layout); keys and values to the pages");
    m.def("min_gru", &min_gru,
          "element-wise gated recurrence with carried fp32 state");
    m.def("mixed_score_attn", &mixed_score_attn,
          "paged windowed GQA attention with capped, head-mixed scores, an "
          "optional sink logit and head gate");
}
