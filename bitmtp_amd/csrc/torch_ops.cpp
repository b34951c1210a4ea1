// libbonsai_torch.so: the packed GEMV and its activation quantiser as registered PyTorch
// operators (namespace "bonsai"), for callers that want dispatcher ops -- fake-tensor shape
// inference, torch.compile, no Python between the tensors and the C ABI -- instead of the ctypes
// binding.  Host code only: every operator checks its tensors, allocates the result with
// PyTorch's allocator and hands plain pointers plus the current stream to the C ABI of
// libbonsai_t2.so / libbonsai_q1.so / libbonsai_actq.so (include/bonsai_gemv.h).
//
// Signatures follow the reference's Python operators (src/bonsai_sft/gpu/model.py:118-268):
//   bonsai::t2g128_int8xint2_linear(a_int8 [.., K], b_packed int8 [N, K/4], s f32 [.., 1],
//                                   ws bf16 [N, K/128]) -> bf16 [.., N]
//   bonsai::q1g128_int8xint1_linear(a_int8 [.., K], b_packed int8 [N, K/8], s, ws) -> bf16 [.., N]
//   bonsai::quant_input(x [.., K]) -> (q int8 [.., K], s f32 [.., 1])      (model.py:632-636)
//   bonsai::fused_norm_quant(x bf16 [.., K], w bf16 [K], eps) -> (q, s)                 (model.py:307-319)
//   bonsai::fused_add_norm_quant(x, residual, w, eps) -> (h bf16 [.., K], q, s)          (model.py:322-336)
//   bonsai::silu_mul_quant(gate_up bf16 [.., 2F]) -> (q int8 [.., F], s f32 [.., 1])     (model.py:1058-1061)
#include <ATen/ATen.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <initializer_list>
#include <tuple>
#include <vector>

#include "../../include/bonsai_gemv.h"

namespace {

void check_gemv_inputs(const char *kind, int bits, const at::Tensor &a, const at::Tensor &b,
                       const at::Tensor &s, const at::Tensor &ws) {
    TORCH_CHECK(a.dim() >= 1 && b.dim() == 2, kind, ": expected rank >= 1 activation and rank-2 weight");
    const int64_t k = b.size(1) * (8 / bits), n = b.size(0);
    TORCH_CHECK(k % 128 == 0 && k >= 128, kind, ": K must be a multiple of 128, got ", k);
    TORCH_CHECK(a.size(-1) == k, kind, ": activation width mismatch: ", a.size(-1), " != ", k);
    TORCH_CHECK(ws.dim() == 2 && ws.size(0) == n && ws.size(1) == k / 128, kind,
                ": invalid weight scale shape");
    TORCH_CHECK(a.scalar_type() == at::kChar && b.scalar_type() == at::kChar &&
                    (ws.scalar_type() == at::kBFloat16 || ws.scalar_type() == at::kHalf),
                kind, ": invalid activation, packed-weight, or scale dtype");
    const int64_t m = a.numel() / k;
    TORCH_CHECK(s.scalar_type() == at::kFloat && s.numel() == m, kind,
                ": activation scales must be float32 with one value per row");
}

template <int BITS>
at::Tensor gemv_cuda(const at::Tensor &a, const at::Tensor &b, const at::Tensor &s,
                     const at::Tensor &ws) {
    const char *kind = BITS == 2 ? "t2g128" : "q1g128";
    check_gemv_inputs(kind, BITS, a, b, s, ws);
    TORCH_CHECK(a.is_cuda() && b.is_cuda() && s.is_cuda() && ws.is_cuda() && a.is_contiguous() &&
                    b.is_contiguous() && s.is_contiguous() && ws.is_contiguous(),
                kind, ": inputs and scales must be contiguous CUDA tensors");
    TORCH_CHECK(b.device() == a.device() && s.device() == a.device() && ws.device() == a.device(),
                kind, ": inputs and scales must share one CUDA device");
    const int64_t n = b.size(0), k = a.size(-1), m = a.numel() / k;
    std::vector<int64_t> shape(a.sizes().begin(), a.sizes().end());
    shape.back() = n;
    at::Tensor out = at::empty(shape, a.options().dtype(at::kBFloat16));
    if (m == 0) return out;
    c10::DeviceGuard guard(a.device());
    void *stream = c10::hip::getCurrentHIPStream().stream();
    const int scale_kind = ws.scalar_type() == at::kHalf ? BONSAI_SCALE_F16 : BONSAI_SCALE_BF16;
    const auto fn = BITS == 2 ? t2g128_gemv_ex : q1g128_gemv_ex;
    const int rc = fn(static_cast<const int8_t *>(a.data_ptr()), static_cast<const uint8_t *>(b.data_ptr()),
                      out.data_ptr(), static_cast<const float *>(s.data_ptr()), ws.data_ptr(), (int)m,
                      (int)n, (int)k, BONSAI_OUT_BF16, scale_kind, stream);
    TORCH_CHECK(rc == 0, kind, ": native GEMV returned status ", rc, " for M=", m, " N=", n, " K=", k);
    return out;
}

template <int BITS>
at::Tensor gemv_meta(const at::Tensor &a, const at::Tensor &b, const at::Tensor &s,
                     const at::Tensor &ws) {
    check_gemv_inputs(BITS == 2 ? "t2g128" : "q1g128", BITS, a, b, s, ws);
    std::vector<int64_t> shape(a.sizes().begin(), a.sizes().end());
    shape.back() = b.size(0);
    return at::empty(shape, a.options().dtype(at::kBFloat16));
}

int x_kind_of(const at::Tensor &x) {
    switch (x.scalar_type()) {
        case at::kBFloat16: return BONSAI_X_BF16;
        case at::kHalf: return BONSAI_X_F16;
        case at::kFloat: return BONSAI_X_F32;
        default: TORCH_CHECK(false, "quant_input: expected a bf16, fp16 or fp32 tensor");
    }
    return -1;
}

std::tuple<at::Tensor, at::Tensor> quant_shapes(const at::Tensor &x) {
    TORCH_CHECK(x.dim() >= 1 && x.size(-1) >= 1, "quant_input: expected rank >= 1");
    x_kind_of(x);
    std::vector<int64_t> sshape(x.sizes().begin(), x.sizes().end());
    sshape.back() = 1;
    return {at::empty(x.sizes(), x.options().dtype(at::kChar)),
            at::empty(sshape, x.options().dtype(at::kFloat))};
}

std::tuple<at::Tensor, at::Tensor> quant_input_cuda(const at::Tensor &x) {
    TORCH_CHECK(x.is_cuda() && x.is_contiguous(), "quant_input: expected a contiguous CUDA tensor");
    auto [q, s] = quant_shapes(x);
    const int64_t k = x.size(-1), m = x.numel() / k;
    if (m == 0) return {q, s};
    c10::DeviceGuard guard(x.device());
    void *stream = c10::hip::getCurrentHIPStream().stream();
    const int rc = bonsai_act_quant_int8(x.data_ptr(), x_kind_of(x), static_cast<int8_t *>(q.data_ptr()),
                                         static_cast<float *>(s.data_ptr()), (int)m, (int)k, stream);
    TORCH_CHECK(rc == 0, "quant_input: native quantiser returned status ", rc);
    return {q, s};
}

std::tuple<at::Tensor, at::Tensor> quant_input_meta(const at::Tensor &x) { return quant_shapes(x); }

// ---- fused producers ---------------------------------------------------------------------
void check_bf16_rows(const char *op, const at::Tensor &x, const at::Tensor &w) {
    TORCH_CHECK(x.dim() >= 1 && x.scalar_type() == at::kBFloat16, op, ": expected a bf16 tensor of rank >= 1");
    const int64_t k = x.size(-1);
    TORCH_CHECK(k >= 8 && k % 8 == 0, op, ": the last dimension must be a multiple of 8");
    TORCH_CHECK(w.scalar_type() == at::kBFloat16 && w.dim() == 1 && w.size(0) == k, op, ": weight must be bf16 [K]");
}

std::vector<int64_t> with_last(const at::Tensor &x, int64_t last) {
    std::vector<int64_t> shape(x.sizes().begin(), x.sizes().end());
    shape.back() = last;
    return shape;
}

void check_cuda_contiguous(const char *op, std::initializer_list<const at::Tensor *> ts) {
    const at::Tensor *first = *ts.begin();
    for (const at::Tensor *t : ts)
        TORCH_CHECK(t->is_cuda() && t->is_contiguous() && t->device() == first->device(), op,
                    ": expected contiguous CUDA tensors on one device");
}

std::tuple<at::Tensor, at::Tensor> norm_quant_meta(const at::Tensor &x, const at::Tensor &w, double) {
    check_bf16_rows("fused_norm_quant", x, w);
    return {at::empty(x.sizes(), x.options().dtype(at::kChar)),
            at::empty(with_last(x, 1), x.options().dtype(at::kFloat))};
}

std::tuple<at::Tensor, at::Tensor> norm_quant_cuda(const at::Tensor &x, const at::Tensor &w, double eps) {
    auto [q, s] = norm_quant_meta(x, w, eps);
    check_cuda_contiguous("fused_norm_quant", {&x, &w});
    const int64_t k = x.size(-1), m = x.numel() / k;
    if (m == 0) return {q, s};
    c10::DeviceGuard guard(x.device());
    const int rc = bonsai_rmsnorm_quant_int8(x.data_ptr(), w.data_ptr(), (float)eps, static_cast<int8_t *>(q.data_ptr()),
                                             static_cast<float *>(s.data_ptr()), (int)m, (int)k,
                                             c10::hip::getCurrentHIPStream().stream());
    TORCH_CHECK(rc == 0, "fused_norm_quant: native launch failed with status ", rc);
    return {q, s};
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> add_norm_quant_meta(const at::Tensor &x, const at::Tensor &residual,
                                                                   const at::Tensor &w, double) {
    check_bf16_rows("fused_add_norm_quant", x, w);
    TORCH_CHECK(residual.scalar_type() == at::kBFloat16 && residual.sizes() == x.sizes(),
                "fused_add_norm_quant: residual must match x");
    return {at::empty(x.sizes(), x.options()), at::empty(x.sizes(), x.options().dtype(at::kChar)),
            at::empty(with_last(x, 1), x.options().dtype(at::kFloat))};
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> add_norm_quant_cuda(const at::Tensor &x, const at::Tensor &residual,
                                                                   const at::Tensor &w, double eps) {
    auto [h, q, s] = add_norm_quant_meta(x, residual, w, eps);
    check_cuda_contiguous("fused_add_norm_quant", {&x, &residual, &w});
    const int64_t k = x.size(-1), m = x.numel() / k;
    if (m == 0) return {h, q, s};
    c10::DeviceGuard guard(x.device());
    const int rc = bonsai_add_rmsnorm_quant_int8(x.data_ptr(), residual.data_ptr(), w.data_ptr(), (float)eps,
                                                 h.data_ptr(), static_cast<int8_t *>(q.data_ptr()),
                                                 static_cast<float *>(s.data_ptr()), (int)m, (int)k,
                                                 c10::hip::getCurrentHIPStream().stream());
    TORCH_CHECK(rc == 0, "fused_add_norm_quant: native launch failed with status ", rc);
    return {h, q, s};
}

std::tuple<at::Tensor, at::Tensor> silu_mul_quant_meta(const at::Tensor &gate_up) {
    TORCH_CHECK(gate_up.dim() >= 1 && gate_up.scalar_type() == at::kBFloat16,
                "silu_mul_quant: expected a bf16 tensor of rank >= 1");
    const int64_t f2 = gate_up.size(-1);
    TORCH_CHECK(f2 >= 16 && f2 % 16 == 0, "silu_mul_quant: last dimension must be 2F with F a multiple of 8");
    return {at::empty(with_last(gate_up, f2 / 2), gate_up.options().dtype(at::kChar)),
            at::empty(with_last(gate_up, 1), gate_up.options().dtype(at::kFloat))};
}

std::tuple<at::Tensor, at::Tensor> silu_mul_quant_cuda(const at::Tensor &gate_up) {
    auto [q, s] = silu_mul_quant_meta(gate_up);
    check_cuda_contiguous("silu_mul_quant", {&gate_up});
    const int64_t f2 = gate_up.size(-1), m = gate_up.numel() / f2;
    if (m == 0) return {q, s};
    c10::DeviceGuard guard(gate_up.device());
    const int rc = bonsai_silu_mul_quant_int8(gate_up.data_ptr(), static_cast<int8_t *>(q.data_ptr()),
                                              static_cast<float *>(s.data_ptr()), (int)m, (int)(f2 / 2),
                                              c10::hip::getCurrentHIPStream().stream());
    TORCH_CHECK(rc == 0, "silu_mul_quant: native launch failed with status ", rc);
    return {q, s};
}

}  // namespace

TORCH_LIBRARY(bonsai, m) {
    m.def("t2g128_int8xint2_linear(Tensor a_int8, Tensor b_packed, Tensor s, Tensor ws) -> Tensor");
    m.def("q1g128_int8xint1_linear(Tensor a_int8, Tensor b_packed, Tensor s, Tensor ws) -> Tensor");
    m.def("quant_input(Tensor x) -> (Tensor, Tensor)");
    m.def("fused_norm_quant(Tensor x, Tensor w, float eps) -> (Tensor, Tensor)");
    m.def("fused_add_norm_quant(Tensor x, Tensor residual, Tensor w, float eps) -> (Tensor, Tensor, Tensor)");
    m.def("silu_mul_quant(Tensor gate_up) -> (Tensor, Tensor)");
}

TORCH_LIBRARY_IMPL(bonsai, CUDA, m) {
    m.impl("t2g128_int8xint2_linear", &gemv_cuda<2>);
    m.impl("q1g128_int8xint1_linear", &gemv_cuda<1>);
    m.impl("quant_input", &quant_input_cuda);
    m.impl("fused_norm_quant", &norm_quant_cuda);
    m.impl("fused_add_norm_quant", &add_norm_quant_cuda);
    m.impl("silu_mul_quant", &silu_mul_quant_cuda);
}

TORCH_LIBRARY_IMPL(bonsai, Meta, m) {
    m.impl("t2g128_int8xint2_linear", &gemv_meta<2>);
    m.impl("q1g128_int8xint1_linear", &gemv_meta<1>);
    m.impl("quant_input", &quant_input_meta);
    m.impl("fused_norm_quant", &norm_quant_meta);
    m.impl("fused_add_norm_quant", &add_norm_quant_meta);
    m.impl("silu_mul_quant", &silu_mul_quant_meta);
}
