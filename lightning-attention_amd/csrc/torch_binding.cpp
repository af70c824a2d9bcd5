// PyTorch operators over the C ABI of liblightning_attn_hip.so, as C++ autograd functions.
//
// The Python operators in lightning_attn/ops/hip do the same work through ctypes and
// torch.autograd.Function; what they cost on the host (about 120 us for a forward + backward step, most of it
// the Python-side autograd node and its hand-over to the engine's device thread) bounds every step whose kernels
// take less than that.  Here the autograd nodes are C++: the same checks, the same tensor preparation (tensors
// the kernels can address are used in place, others copied), the same entry points.  PyTorch is plumbing
// only: allocation, streams, the autograd graph.  The Python operators use this library when it is built and
// fall back to their own path when it is not; arguments they would reject never reach it.
//
//   lightning_attn_hip::attn(q, k, v, s?, chunks, scan, wide, paired, once, save_states) -> o
//       lightning_attn2 / lightning_attn2_no_decay (lightning_attn/ops/triton/lightning_attn2.py:398-507,
//       lightning_attn2_no_decay.py:367-471)
//   lightning_attn_hip::srmsnorm(x, eps) -> y
//       _SrmsNorm (lightning_attn/ops/triton/srmsnorm.py:76-175)
//   lightning_attn_hip::attn_silu(q, k, v, s?, chunks, scan, wide, paired, once) -> o      (no backward pass)
//   lightning_attn_hip::norm_gate(o, g, weight, bias, eps) -> y
//       the attention block's activation and gated output norm (examples/module/tnl_attn.py:51-54, 66-69)
#include <ATen/ATen.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/csrc/autograd/custom_function.h>
#include <torch/library.h>

#include "lightning_attn_hip.h"

namespace {

using at::Tensor;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

int dtype_code(at::ScalarType t) {
    switch (t) {
        case at::kBFloat16: return LA_BF16;
        case at::kHalf: return LA_FP16;
        case at::kFloat: return LA_FP32;
        default: TORCH_CHECK_TYPE(false, "unsupported dtype ", t, " (bfloat16, float16 or float32)");
    }
}

void check(int rc, const char* what) {
    TORCH_CHECK(rc == 0, what, " failed: ", la_error_string(rc), " (code ", rc, ")");
}

void* stream_of(const Tensor& t) { return c10::hip::getCurrentHIPStream(t.device().index()).stream(); }

// (batch, head, token) strides of a 4-d tensor; those of size-1 dims (never used for addressing, may be anything)
// replaced by the dense value
void norm_strides(const Tensor& t, int64_t* st) {
    for (int i = 0; i < 4; ++i) st[i] = t.stride(i);
    for (int i = 2; i >= 0; --i)
        if (t.size(i) == 1) st[i] = t.size(i + 1) * st[i + 1];
}

// the kernels can address `t` (b, h, n, c) through its own strides
bool in_place_ok(const Tensor& t) {
    if (t.scalar_type() == at::kFloat || t.dim() != 4 || t.stride(3) != 1) return false;
    const int64_t elt = t.element_size();
    if (reinterpret_cast<uintptr_t>(t.data_ptr()) % 16) return false;
    int64_t st[4];
    norm_strides(t, st);
    for (int i = 0; i < 3; ++i)
        if (st[i] <= 0 || (st[i] * elt) % 16) return false;
    if (st[2] < t.size(3)) return false;
    return ((t.size(2) - 1) * st[2] + t.size(3)) * elt < (int64_t(1) << 31);
}

// `t` itself where the kernels can address it, else a dense, 16-byte aligned copy
Tensor usable(const Tensor& t) {
    if (t.is_contiguous())
        return reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0 ? t : t.clone(at::MemoryFormat::Contiguous);
    return in_place_ok(t) ? t : t.contiguous();
}

struct Opts {
    la_launch_opts o;
    bool given, save_states;
};
Opts make_opts(int64_t chunks, int64_t scan, int64_t wide, int64_t paired, int64_t once, bool save_states) {
    Opts r;
    r.o = la_launch_opts{(int32_t)chunks, (int32_t)scan, (int32_t)wide, (int32_t)paired, (int32_t)once};
    r.given = chunks || scan || wide || paired || once;
    r.save_states = save_states;
    return r;
}

struct Attn : public torch::autograd::Function<Attn> {
    static Tensor forward(AutogradContext* ctx, const Tensor& q_in, const Tensor& k_in, const Tensor& v_in,
                          const c10::optional<Tensor>& s_in, int64_t chunks, int64_t scan, int64_t wide, int64_t paired,
                          int64_t once, bool save_states) {
        const Opts op = make_opts(chunks, scan, wide, paired, once, save_states);
        const Tensor q = usable(q_in), k = usable(k_in), v = usable(v_in);
        const int64_t b = q.size(0), h = q.size(1), n = q.size(2), d = q.size(3), e = v.size(3);
        Tensor s;
        if (s_in.has_value() && s_in->defined()) {
            s = *s_in;
            if (s.scalar_type() != at::kFloat || s.device() != q.device() || !s.is_contiguous())
                s = s.to(q.device(), at::kFloat).contiguous();
        }
        const int code = dtype_code(q.scalar_type());
        const la_launch_opts* lo = op.given ? &op.o : nullptr;
        Tensor o = at::empty_like(v);  // same sizes as v; dense, in v's memory order
        const c10::DeviceGuard guard(q.device());
        const size_t ws_bytes = la_workspace_bytes_opts(0, b, h, n, d, e, code, lo);
        Tensor ws, saved;
        if (ws_bytes) ws = at::empty({(int64_t)ws_bytes}, q.options().dtype(at::kByte));
        // (save_states arrives false when no backward pass can follow)
        const size_t sv_bytes = op.save_states ? la_saved_state_bytes(b, h, n, d, e, code, lo) : 0;
        if (sv_bytes) saved = at::empty({(int64_t)(sv_bytes / 4)}, q.options().dtype(at::kFloat));
        int64_t st[4][4], strides[12];
        const bool dense = q.is_contiguous() && k.is_contiguous() && v.is_contiguous() && o.is_contiguous();
        if (!dense) {
            const Tensor* ts[4] = {&q, &k, &v, &o};
            for (int i = 0; i < 4; ++i) {
                norm_strides(*ts[i], st[i]);
                for (int j = 0; j < 3; ++j) strides[3 * i + j] = st[i][j];
            }
        }
        check(la_fwd_save(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.defined() ? s.data_ptr<float>() : nullptr, o.data_ptr(),
                          dense ? nullptr : strides, b, h, n, d, e, code, ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, lo,
                          sv_bytes ? saved.data_ptr<float>() : nullptr, sv_bytes, stream_of(q)),
              "la_fwd");
        ctx->save_for_backward({q, k, v, s, saved});
        ctx->saved_data["opts"] = std::vector<int64_t>{chunks, scan, wide, paired, once};
        return o;
    }

    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const auto sv = ctx->get_saved_variables();
        const Tensor &q = sv[0], &k = sv[1], &v = sv[2], &s = sv[3], &saved = sv[4];
        const auto ov = ctx->saved_data["opts"].toIntVector();
        const Opts op = make_opts(ov[0], ov[1], ov[2], ov[3], ov[4], true);
        const la_launch_opts* lo = op.given ? &op.o : nullptr;
        const int64_t b = q.size(0), h = q.size(1), n = q.size(2), d = q.size(3), e = v.size(3);
        Tensor dout = grads[0];
        TORCH_CHECK(dout.defined(), "lightning_attn2 backward: no upstream gradient");
        TORCH_CHECK(dout.device() == q.device(), "lightning_attn2 backward: the upstream gradient is on ", dout.device(),
                    ", the inputs on ", q.device());
        if (dout.scalar_type() != q.scalar_type()) dout = dout.to(q.scalar_type());
        dout = usable(dout);
        const int code = dtype_code(q.scalar_type());
        Tensor dq = at::empty_like(q), dk = at::empty_like(k), dv = at::empty_like(v);
        const c10::DeviceGuard guard(q.device());
        const size_t ws_bytes = la_workspace_bytes_opts(1, b, h, n, d, e, code, lo);
        Tensor ws;
        if (ws_bytes) ws = at::empty({(int64_t)ws_bytes}, q.options().dtype(at::kByte));
        const Tensor* ts[7] = {&q, &k, &v, &dout, &dq, &dk, &dv};
        bool dense = true;
        for (const Tensor* t : ts) dense = dense && t->is_contiguous();
        int64_t st[4], strides[21];
        if (!dense)
            for (int i = 0; i < 7; ++i) {
                norm_strides(*ts[i], st);
                for (int j = 0; j < 3; ++j) strides[3 * i + j] = st[j];
            }
        const size_t sv_bytes = saved.defined() ? (size_t)saved.numel() * 4 : 0;
        check(la_bwd_saved(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.defined() ? s.data_ptr<float>() : nullptr, dout.data_ptr(),
                           dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dense ? nullptr : strides, b, h, n, d, e, code,
                           ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, lo, sv_bytes ? saved.data_ptr<float>() : nullptr, sv_bytes,
                           stream_of(q)),
              "la_bwd");
        return {dq, dk, dv, Tensor(), Tensor(), Tensor(), Tensor(), Tensor(), Tensor(), Tensor()};
    }
};

Tensor attn(const Tensor& q, const Tensor& k, const Tensor& v, const c10::optional<Tensor>& s, int64_t chunks, int64_t scan,
            int64_t wide, int64_t paired, int64_t once, bool save_states) {
    // states for the backward pass only where one can follow (inside forward() gradient mode is off)
    const bool for_backward = at::GradMode::is_enabled() && (q.requires_grad() || k.requires_grad() || v.requires_grad());
    return Attn::apply(q, k, v, s, chunks, scan, wide, paired, once, save_states && for_backward);
}

struct SrmsNorm : public torch::autograd::Function<SrmsNorm> {
    static Tensor forward(AutogradContext* ctx, const Tensor& x, double eps) {
        // eps too small for fp16 (srmsnorm.py:80-81)
        if (x.scalar_type() == at::kHalf && eps < 1.6e-5) eps = 1.6e-5;
        Tensor x2 = x.reshape({-1, x.size(-1)});
        if (!x2.is_contiguous()) x2 = x2.contiguous();
        const int64_t rows = x2.size(0), cols = x2.size(1);
        // same bound as the reference: one row may not exceed 64 KB (srmsnorm.py:94-97)
        TORCH_CHECK(cols <= 65536 / (int64_t)x.element_size(), "This layer norm doesn't support feature dim >= 64KB.");
        Tensor y = at::empty_like(x2);
        Tensor rstd = at::empty({rows}, x.options().dtype(at::kFloat));
        const c10::DeviceGuard guard(x.device());
        check(srmsnorm_fwd(x2.data_ptr(), y.data_ptr(), rstd.data_ptr<float>(), rows, cols, rows > 1 ? x2.stride(0) : cols,
                           (float)eps, dtype_code(x.scalar_type()), stream_of(x)),
              "srmsnorm_fwd");
        ctx->save_for_backward({x, rstd});
        return y.reshape(x.sizes());
    }

    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const auto sv = ctx->get_saved_variables();
        const Tensor &x = sv[0], &rstd = sv[1];
        Tensor x2 = x.reshape({-1, x.size(-1)});
        if (!x2.is_contiguous()) x2 = x2.contiguous();
        const int64_t rows = x2.size(0), cols = x2.size(1);
        Tensor dy = grads[0];
        TORCH_CHECK(dy.defined() && dy.device() == x.device(), "SimpleRMSNorm backward: the upstream gradient is not on ", x.device());
        dy = dy.contiguous();
        if (dy.scalar_type() != x.scalar_type()) dy = dy.to(x.scalar_type());
        TORCH_CHECK(dy.numel() == x.numel(),
                    "Something is wrong in the backward graph, possibly because of an inplace operation after the layernorm");
        Tensor dx = at::empty_like(dy);
        const c10::DeviceGuard guard(x.device());
        check(srmsnorm_bwd(x2.data_ptr(), dy.data_ptr(), rstd.data_ptr<float>(), dx.data_ptr(), rows, cols,
                           rows > 1 ? x2.stride(0) : cols, dtype_code(x.scalar_type()), stream_of(x)),
              "srmsnorm_bwd");
        return {dx.reshape(dy.sizes()), Tensor()};
    }
};

Tensor srmsnorm(const Tensor& x, double eps) { return SrmsNorm::apply(x, eps); }

// attention over silu(q), silu(k), silu(v) in one forward kernel; no backward pass (callers check that none is wanted)
Tensor attn_silu(const Tensor& q_in, const Tensor& k_in, const Tensor& v_in, const c10::optional<Tensor>& s_in, int64_t chunks,
                 int64_t scan, int64_t wide, int64_t paired, int64_t once) {
    const Opts op = make_opts(chunks, scan, wide, paired, once, false);
    const Tensor q = usable(q_in.detach()), k = usable(k_in.detach()), v = usable(v_in.detach());
    const int64_t b = q.size(0), h = q.size(1), n = q.size(2), d = q.size(3), e = v.size(3);
    Tensor s;
    if (s_in.has_value() && s_in->defined()) {
        s = s_in->detach();
        if (s.scalar_type() != at::kFloat || s.device() != q.device() || !s.is_contiguous())
            s = s.to(q.device(), at::kFloat).contiguous();
    }
    const int code = dtype_code(q.scalar_type());
    const la_launch_opts* lo = op.given ? &op.o : nullptr;
    Tensor o = at::empty_like(v);
    const c10::DeviceGuard guard(q.device());
    const size_t ws_bytes = la_workspace_bytes_opts(0, b, h, n, d, e, code, lo);
    Tensor ws;
    if (ws_bytes) ws = at::empty({(int64_t)ws_bytes}, q.options().dtype(at::kByte));
    int64_t st[4], strides[12];
    const bool dense = q.is_contiguous() && k.is_contiguous() && v.is_contiguous() && o.is_contiguous();
    if (!dense) {
        const Tensor* ts[4] = {&q, &k, &v, &o};
        for (int i = 0; i < 4; ++i) {
            norm_strides(*ts[i], st);
            for (int j = 0; j < 3; ++j) strides[3 * i + j] = st[j];
        }
    }
    check(la_fwd_silu(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.defined() ? s.data_ptr<float>() : nullptr, o.data_ptr(),
                      dense ? nullptr : strides, b, h, n, d, e, code, ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, lo, stream_of(q)),
          "la_fwd_silu");
    return o;
}

// row-major and 16-byte aligned (a dense view into a larger buffer may start off that grid)
Tensor dense_rows(const Tensor& t) {
    const Tensor c = t.is_contiguous() ? t : t.contiguous();
    return reinterpret_cast<uintptr_t>(c.data_ptr()) % 16 == 0 ? c : c.clone();
}

// layer_norm(o; weight, bias, eps) * sigmoid(g) over the last dim (examples/module/tnl_attn.py:66-69 of the reference)
struct NormGate : public torch::autograd::Function<NormGate> {
    static Tensor forward(AutogradContext* ctx, const Tensor& o, const Tensor& g, const Tensor& weight_in, const Tensor& bias_in,
                          double eps) {
        const int64_t cols = o.size(-1);
        const Tensor o2 = dense_rows(o.reshape({-1, cols})), g2 = dense_rows(g.reshape({-1, cols}));
        const Tensor weight = dense_rows(weight_in), bias = dense_rows(bias_in);
        const int64_t rows = o2.size(0);
        Tensor y = at::empty_like(o2);
        Tensor mean = at::empty({rows}, o.options().dtype(at::kFloat)), rstd = at::empty({rows}, o.options().dtype(at::kFloat));
        const c10::DeviceGuard guard(o.device());
        check(norm_gate_fwd(o2.data_ptr(), g2.data_ptr(), weight.data_ptr(), bias.data_ptr(), y.data_ptr(), mean.data_ptr<float>(),
                            rstd.data_ptr<float>(), rows, cols, (float)eps, dtype_code(o.scalar_type()), stream_of(o)),
              "norm_gate_fwd");
        ctx->save_for_backward({o2, g2, weight, bias, mean, rstd});
        ctx->saved_data["shape"] = o.sizes().vec();
        return y.reshape(o.sizes());
    }

    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const auto sv = ctx->get_saved_variables();
        const Tensor &o2 = sv[0], &g2 = sv[1], &weight = sv[2], &bias = sv[3], &mean = sv[4], &rstd = sv[5];
        const auto shape = ctx->saved_data["shape"].toIntVector();
        const int64_t rows = o2.size(0), cols = o2.size(1);
        Tensor dy = grads[0];
        TORCH_CHECK(dy.defined() && dy.device() == o2.device(), "norm_gate backward: the upstream gradient is not on ", o2.device());
        if (dy.scalar_type() != o2.scalar_type()) dy = dy.to(o2.scalar_type());
        const Tensor dy2 = dense_rows(dy.reshape({rows, cols}));
        const int code = dtype_code(o2.scalar_type());
        Tensor d_o = at::empty_like(o2), d_g = at::empty_like(g2), dw = at::empty_like(weight), db = at::empty_like(bias);
        const c10::DeviceGuard guard(o2.device());
        const size_t ws_bytes = norm_gate_workspace_bytes(rows, cols, code);
        Tensor ws = at::empty({(int64_t)std::max<size_t>(ws_bytes, 4)}, o2.options().dtype(at::kByte));
        check(norm_gate_bwd(o2.data_ptr(), g2.data_ptr(), weight.data_ptr(), bias.data_ptr(), mean.data_ptr<float>(),
                            rstd.data_ptr<float>(), dy2.data_ptr(), d_o.data_ptr(), d_g.data_ptr(), dw.data_ptr(), db.data_ptr(),
                            ws.data_ptr(), ws_bytes, rows, cols, code, stream_of(o2)),
              "norm_gate_bwd");
        return {d_o.reshape(shape), d_g.reshape(shape), dw, db, Tensor()};
    }
};

Tensor norm_gate(const Tensor& o, const Tensor& g, const Tensor& weight, const Tensor& bias, double eps) {
    return NormGate::apply(o, g, weight, bias, eps);
}

}  // namespace

TORCH_LIBRARY(lightning_attn_hip, m) {
    m.def("attn", &attn);
    m.def("srmsnorm", &srmsnorm);
    m.def("attn_silu", &attn_silu);
    m.def("norm_gate", &norm_gate);
}
