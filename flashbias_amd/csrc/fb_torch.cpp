// The operator's autograd function in C++: what flashbias_amd/interface.py does per call (argument
// checks of _flash_attn_forward / _flash_attn_backward, flash_bias/flash_bias_triton.py:1100-1143 and
// :1197-1231, the parameter block, the output allocations, the launch on torch's current stream, the
// reduction of broadcast factors' gradients) without the interpreter in the way: at sequence lengths
// of a few thousand the kernels of a forward + backward take 50-150 us, which is what the Python
// path costs on the host.  Everything that touches the GPU still goes through the C ABI of
// include/flashbias.h; torch provides memory, the stream and the autograd graph.
//
// Expects kernel-ready inputs (flash_bias_func in interface.py prepares the rare cases with ordinary
// differentiable tensor operations before calling in): q, k, v (B, L, H, d); factors (B|1, L, H|1, r)
// or none; additive mask (B|1, H|1, 1|Lq, Lk) or none.
#include <torch/extension.h>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <cmath>
#include <cstring>

#include "flashbias.h"

namespace {

using torch::Tensor;
using torch::autograd::AutogradContext;
using torch::autograd::tensor_list;

fb_tensor t4(const Tensor &x) { return fb_tensor{x.data_ptr(), x.stride(0), x.stride(2), x.stride(1)}; }

Tensor channel_contiguous(const Tensor &x) { return x.stride(-1) == 1 ? x : x.contiguous(); }

int dtype_code(c10::ScalarType t) {
    if (t == torch::kFloat16) return FB_F16;
    if (t == torch::kBFloat16) return FB_BF16;
    if (t == torch::kFloat32) return FB_F32;
    TORCH_CHECK(false, "unsupported dtype ", t);
}

void check(int status) { TORCH_CHECK(status == FB_OK, "flashbias status ", status, ": ", fb_last_error()); }

// The parameter block shared by forward and backward.  `keep` receives the expanded views whose
// data the block points at.
fb_params block(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor &qb, const Tensor &kb, const Tensor &mask,
                bool causal, double scale, tensor_list &keep) {
    TORCH_CHECK(q.dim() == 4 && k.dim() == 4 && v.dim() == 4, "q, k, v must be (batch, seqlen, nheads, headdim)");
    const int64_t B = q.size(0), Lq = q.size(1), H = q.size(2), d = q.size(3), Lk = k.size(1);
    TORCH_CHECK(k.size(0) == B && k.size(2) == H && k.size(3) == d && v.sizes() == k.sizes(), "k, v must be (batch, seqlen_k, nheads, headdim)");
    TORCH_CHECK(d <= FB_MAX_HEADDIM, "FlashBias only supports head dimensions up to 128");
    TORCH_CHECK(q.scalar_type() == k.scalar_type() && q.scalar_type() == v.scalar_type(), "All tensors must have the same type");
    TORCH_CHECK(q.scalar_type() == torch::kFloat16 || q.scalar_type() == torch::kBFloat16, "Only support fp16 and bf16");
    TORCH_CHECK(q.is_cuda() && k.is_cuda() && v.is_cuda(), "q, k, v must be on the GPU");
    fb_params p;
    std::memset(&p, 0, sizeof(p));
    p.size = sizeof(p);
    p.dtype = dtype_code(q.scalar_type());
    p.B = (int32_t)B; p.H = (int32_t)H; p.Lq = (int32_t)Lq; p.Lk = (int32_t)Lk; p.d = (int32_t)d;
    p.causal = causal ? 1 : 0;
    p.scale = (float)scale;
    p.q = t4(q); p.k = t4(k); p.v = t4(v);
    if (qb.defined()) {
        TORCH_CHECK(kb.defined() && qb.scalar_type() == q.scalar_type() && kb.scalar_type() == q.scalar_type() && qb.is_cuda() &&
                        kb.is_cuda() && qb.dim() == 4 && kb.dim() == 4 && qb.size(3) == kb.size(3),
                    "q_bias, k_bias must be GPU tensors of the input dtype and one rank");
        const int64_t r = qb.size(3);
        // stride-0 broadcast over batch / heads (flash_bias_triton.py:1135-1136)
        const Tensor qe = qb.expand({B, Lq, H, r}), ke = kb.expand({B, Lk, H, r});
        p.r = (int32_t)r;
        p.q_bias = t4(qe);
        p.k_bias = t4(ke);
        keep.push_back(qe);
        keep.push_back(ke);
    }
    if (mask.defined()) {
        TORCH_CHECK(mask.dim() == 4 && mask.is_cuda() && (mask.scalar_type() == q.scalar_type() || mask.scalar_type() == torch::kFloat32),
                    "mask must be a 4-d GPU tensor of the input dtype or fp32");
        if (mask.size(2) == 1 && mask.size(3) == Lk)
            p.mask_type = FB_MASK_VECTOR;
        else if (mask.size(2) == Lq && mask.size(3) == Lk)
            p.mask_type = FB_MASK_MATRIX;
        else
            TORCH_CHECK(false, "Last 2 dimensions of mask must be (1, seqlen_k) or (seqlen_q, seqlen_k)");
        const Tensor me = mask.expand({B, H, Lq, Lk});
        p.mask = fb_tensor{me.data_ptr(), me.stride(0), me.stride(1), me.stride(2)};
        p.mask_dtype = dtype_code(mask.scalar_type());
        keep.push_back(me);
    }
    return p;
}

// The gradient of `ref` from the full (B, L, H, r) gradient the kernels wrote: summed over the dims in
// which `ref` was broadcast, in fp32 (over the batch by the library's streaming kernel).
Tensor reduce_like(Tensor full, const Tensor &ref, hipStream_t stream) {
    bool over_batch = ref.size(0) == 1 && full.size(0) != 1;
    const bool over_heads = ref.size(2) == 1 && full.size(2) != 1;
    const int64_t n = full.size(1) * full.size(2) * full.size(3);
    if (over_batch && full.is_contiguous() && n % 8 == 0) {
        Tensor out = torch::empty({1, full.size(1), full.size(2), full.size(3)},
                                  full.options().dtype(over_heads ? torch::kFloat32 : full.scalar_type()));
        check(fb_sum_over_batch(full.data_ptr(), out.data_ptr(), dtype_code(full.scalar_type()), dtype_code(out.scalar_type()),
                                full.size(0), n, n, stream));
        full = out;
        over_batch = false;
    }
    if (over_batch || over_heads) {
        std::vector<int64_t> dims;
        if (over_batch) dims.push_back(0);
        if (over_heads) dims.push_back(2);
        full = full.sum(dims, /*keepdim=*/true, torch::kFloat32);
    }
    if (full.scalar_type() != ref.scalar_type()) full = full.to(ref.scalar_type());
    return full.is_contiguous() ? full : full.contiguous();
}

struct FlashBiasFn : public torch::autograd::Function<FlashBiasFn> {
    static Tensor forward(AutogradContext *ctx, const Tensor &q_in, const Tensor &k_in, const Tensor &v_in,
                          const c10::optional<Tensor> &qb_in, const c10::optional<Tensor> &kb_in,
                          const c10::optional<Tensor> &mask_in, bool causal, double softmax_scale) {
        const Tensor q = channel_contiguous(q_in), k = channel_contiguous(k_in), v = channel_contiguous(v_in);
        Tensor qb, kb, mask;
        if (qb_in.has_value() && qb_in->defined()) {
            TORCH_CHECK(kb_in.has_value() && kb_in->defined(), "q_bias without k_bias");
            qb = channel_contiguous(*qb_in);
            kb = channel_contiguous(*kb_in);
        }
        if (mask_in.has_value() && mask_in->defined()) mask = channel_contiguous(*mask_in);
        const double scale = softmax_scale != 0.0 ? softmax_scale : 1.0 / std::sqrt((double)q.size(3));
        tensor_list keep;
        fb_params p = block(q, k, v, qb, kb, mask, causal, scale, keep);
        Tensor o = torch::empty_like(q);
        Tensor lse = torch::empty({q.size(0), q.size(2), q.size(1)}, q.options().dtype(torch::kFloat32));
        p.o = t4(o);
        p.lse = lse.data_ptr<float>();
        {
            const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device()); // (torch on ROCm presents its devices as "cuda")
            check(fb_fwd(&p, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(q.device().index()).stream()));
        }
        ctx->save_for_backward({q, k, v, o, lse, qb, kb, mask});
        ctx->saved_data["causal"] = causal;
        ctx->saved_data["scale"] = scale;
        return o;
    }

    static tensor_list backward(AutogradContext *ctx, tensor_list grads) {
        const auto saved = ctx->get_saved_variables();
        const Tensor &q = saved[0], &k = saved[1], &v = saved[2], &o = saved[3], &lse = saved[4];
        const Tensor &qb = saved[5], &kb = saved[6], &mask = saved[7];
        // as the reference, only a backward that is asked for the mask's gradient fails (flash_bias_triton.py:1371).
        // (The graph edges count the tensor arguments that were given: q, k, v, then the factors, then the mask.)
        if (mask.defined())
            TORCH_CHECK(!ctx->needs_input_grad(qb.defined() ? 5 : 3), "FlashBias does not support mask gradient yet");
        const bool causal = ctx->saved_data["causal"].toBool();
        const double scale = ctx->saved_data["scale"].toDouble();
        const Tensor dout = channel_contiguous(grads[0]);
        tensor_list keep;
        fb_params p = block(q, k, v, qb, kb, mask, causal, scale, keep);
        Tensor dq = torch::empty_like(q), dk = torch::empty_like(k), dv = torch::empty_like(v);
        p.o = t4(o);
        p.lse = lse.data_ptr<float>();
        p.dout = t4(dout);
        p.dq = t4(dq); p.dk = t4(dk); p.dv = t4(dv);
        Tensor dqb_full, dkb_full;
        // (neither factor asks for its gradient: constant factors; the library then skips them)
        const bool factor_grads = p.r && (ctx->needs_input_grad(3) || ctx->needs_input_grad(4));
        // factors shared by a large batch of short sequences: a workgroup walks `group` batch entries (it then loads
        // the factor operand it keeps once), sums their factor gradients itself, and the full-shape tensors shrink by
        // that factor
        // (only for factors saved with a batch of one: a factor expanded over the batch by its caller also has batch
        // stride 0, but autograd wants its gradient in the expanded shape)
        const bool shared = p.r && qb.size(0) == 1 && kb.size(0) == 1 && p.B > 1;
        const int group = p.bias_grad_group = p.r ? (shared ? fb_suggest_bias_grad_group(&p) : 1) : 0;
        if (factor_grads) {
            const int64_t rows = ((int64_t)p.B + group - 1) / group;
            dqb_full = torch::empty({rows, p.Lq, p.H, p.r}, q.options());
            dkb_full = torch::empty({rows, p.Lk, p.H, p.r}, q.options());
            p.dq_bias = t4(dqb_full);
            p.dk_bias = t4(dkb_full);
        }
        // scratch of the backward, sized by the library
        Tensor scratch = torch::empty({(int64_t)(fb_bwd_workspace_bytes(&p) / 4)}, q.options().dtype(torch::kFloat32));
        p.delta = scratch.data_ptr<float>();
        Tensor dqb, dkb;
        {
            const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device()); // (torch on ROCm presents its devices as "cuda")
            const hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(q.device().index()).stream();
            check(fb_bwd(&p, stream));
            if (factor_grads) {
                dqb = reduce_like(dqb_full, qb, stream);
                dkb = reduce_like(dkb_full, kb, stream);
            }
        }
        return {dq, dk, dv, dqb, dkb, Tensor(), Tensor(), Tensor()};
    }
};

// x (..., r) with its last dim zero-padded (or cut) to `rank` columns in one launch of the library; the gradient
// is the same operation the other way.  For contiguous 16-bit GPU tensors (the caller checks).
struct ResizeRankFn : public torch::autograd::Function<ResizeRankFn> {
    static Tensor forward(AutogradContext *ctx, const Tensor &x, int64_t rank) {
        TORCH_CHECK(x.is_cuda() && x.is_contiguous() && x.element_size() == 2 && x.dim() >= 1 && x.numel() > 0 && rank > 0,
                    "resize_rank wants a contiguous fp16 / bf16 GPU tensor");
        ctx->saved_data["rank_in"] = x.size(-1);
        auto shape = x.sizes().vec();
        shape.back() = rank;
        Tensor out = torch::empty(shape, x.options());
        const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
        check(fb_resize_rank(x.data_ptr(), out.data_ptr(), out.numel() / rank, (int)x.size(-1), (int)rank,
                             c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(x.device().index()).stream()));
        return out;
    }

    static tensor_list backward(AutogradContext *ctx, tensor_list grads) {
        return {ResizeRankFn::apply(grads[0].contiguous(), ctx->saved_data["rank_in"].toInt()), Tensor()};
    }
};

Tensor resize_rank(const Tensor &x, int64_t rank) { return ResizeRankFn::apply(x, rank); }

Tensor flash_bias(const Tensor &q, const Tensor &k, const Tensor &v, const c10::optional<Tensor> &q_bias,
                  const c10::optional<Tensor> &k_bias, const c10::optional<Tensor> &mask, bool causal, double softmax_scale) {
    return FlashBiasFn::apply(q, k, v, q_bias, k_bias, mask, causal, softmax_scale);
}

} // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "flash_bias_func with its autograd function in C++ (kernel-ready inputs; see flashbias_amd/interface.py)";
    // what this module was compiled against: the caller compares both with the library it loaded
    m.def("abi", []() { return std::make_pair((int)FB_VERSION, (int)sizeof(fb_params)); });
    m.def("resize_rank", &resize_rank, py::arg("x"), py::arg("rank"));
    m.def("flash_bias", &flash_bias, py::arg("q"), py::arg("k"), py::arg("v"), py::arg("q_bias") = py::none(),
          py::arg("k_bias") = py::none(), py::arg("mask") = py::none(), py::arg("causal") = false,
          py::arg("softmax_scale") = 0.0);
}
