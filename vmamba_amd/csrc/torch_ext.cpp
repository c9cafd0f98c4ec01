// selective_scan_cuda_oflex -- the PyTorch extension module the reference probes for
// (classification/models/csms6s.py:9-14) and calls as
//     out, x, *rest = selective_scan_cuda_oflex.fwd(u, delta, A, B, C, D, delta_bias, delta_softplus, 1, oflex)
// (csms6s.py:81).  This is a thin shim: the argument checks and output allocation of the reference's
// selective_scan_fwd (kernels/selective_scan/csrc/selective_scan/cusoflex/selective_scan_oflex.cpp:143-231),
// then one call into the C ABI of libss2d_hip.so on PyTorch's current HIP stream.  No kernel lives here.
// `bwd` does the same for selective_scan_bwd (selective_scan_oflex.cpp:233-355): checks, zeroed accumulators, one
// call into ss2d_selective_scan_bwd, and the delta-group reductions of :347-352.
#include <ATen/hip/HIPContext.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include <vector>

#include "../../include/ss2d_hip.h"

#define CHECK_SHAPE(x, ...) \
    TORCH_CHECK(x.sizes() == torch::IntArrayRef({__VA_ARGS__}), #x " must have shape (" #__VA_ARGS__ ")")

static int dtype_code(at::ScalarType t) {
    switch (t) {
        case at::ScalarType::Float: return SS2D_F32;
        case at::ScalarType::BFloat16: return SS2D_BF16;
        case at::ScalarType::Half: return SS2D_F16;
        default: return -1;
    }
}

static std::vector<at::Tensor> selective_scan_fwd(const at::Tensor &u, const at::Tensor &delta, const at::Tensor &A,
                                                  const at::Tensor &B, const at::Tensor &C,
                                                  const c10::optional<at::Tensor> &D_,
                                                  const c10::optional<at::Tensor> &delta_bias_, bool delta_softplus,
                                                  int nrows, bool out_float) {
    (void)nrows;  // accepted and ignored, as in the reference (selective_scan_oflex.cpp:224-226)
    const auto input_type = u.scalar_type();
    TORCH_CHECK(dtype_code(input_type) >= 0, "selective_scan_fwd not implemented for input type '", toString(input_type), "'");
    TORCH_CHECK(A.scalar_type() == at::ScalarType::Float, "A must be float32");
    TORCH_CHECK(delta.scalar_type() == input_type && B.scalar_type() == input_type && C.scalar_type() == input_type,
                "delta, B, C must have the dtype of u");
    TORCH_CHECK(u.is_cuda() && delta.is_cuda() && A.is_cuda() && B.is_cuda() && C.is_cuda(), "inputs must be GPU tensors");
    TORCH_CHECK(u.dim() == 3 && delta.dim() == 3 && A.dim() == 2 && B.dim() == 4 && C.dim() == 4, "bad tensor ranks");
    TORCH_CHECK(u.stride(-1) == 1 || u.size(-1) == 1);
    TORCH_CHECK(delta.stride(-1) == 1 || delta.size(-1) == 1);

    const int batch_size = u.size(0), dim = u.size(1), seqlen = u.size(2);
    const int dstate = A.size(1), n_groups = B.size(1), delta_dim = delta.size(1);
    TORCH_CHECK(dim % n_groups == 0, "dims should be dividable by n_groups");
    TORCH_CHECK(dim % delta_dim == 0, "dims should be dividable by delta_dim");
    TORCH_CHECK(dstate <= 256, "selective_scan only supports state dimension <= 256");
    CHECK_SHAPE(u, batch_size, dim, seqlen);
    CHECK_SHAPE(delta, batch_size, delta_dim, seqlen);
    CHECK_SHAPE(A, dim, dstate);
    CHECK_SHAPE(B, batch_size, n_groups, dstate, seqlen);
    TORCH_CHECK(B.stride(-1) == 1 || B.size(-1) == 1);
    CHECK_SHAPE(C, batch_size, n_groups, dstate, seqlen);
    TORCH_CHECK(C.stride(-1) == 1 || C.size(-1) == 1);

    at::Tensor D, delta_bias;
    if (D_.has_value()) {
        D = D_.value();
        TORCH_CHECK(D.scalar_type() == at::ScalarType::Float && D.is_cuda());
        TORCH_CHECK(D.stride(-1) == 1 || D.size(-1) == 1);
        CHECK_SHAPE(D, dim);
    }
    if (delta_bias_.has_value()) {
        delta_bias = delta_bias_.value();
        TORCH_CHECK(delta_bias.scalar_type() == at::ScalarType::Float && delta_bias.is_cuda());
        TORCH_CHECK(delta_bias.stride(-1) == 1 || delta_bias.size(-1) == 1);
        CHECK_SHAPE(delta_bias, delta_dim);
    }

    const int n_chunks = (seqlen + SS2D_SCAN_CHUNK - 1) / SS2D_SCAN_CHUNK;
    at::Tensor out = torch::empty({batch_size, dim, seqlen}, u.options().dtype(out_float ? at::ScalarType::Float : input_type));
    at::Tensor x = torch::empty({batch_size, dim, n_chunks, dstate * 2}, u.options().dtype(at::ScalarType::Float));

    ss2d_scan_params p = {};
    p.batch = batch_size; p.dim = dim; p.seqlen = seqlen; p.dstate = dstate; p.n_groups = n_groups; p.delta_dim = delta_dim;
    p.in_dtype = dtype_code(input_type);
    p.out_dtype = dtype_code(out.scalar_type());
    p.delta_softplus = delta_softplus ? 1 : 0;
    p.u = u.data_ptr(); p.delta = delta.data_ptr(); p.A = A.data_ptr(); p.B = B.data_ptr(); p.C = C.data_ptr();
    p.D = D.defined() ? D.data_ptr() : nullptr;
    p.delta_bias = delta_bias.defined() ? delta_bias.data_ptr() : nullptr;
    p.out = out.data_ptr(); p.x = x.data_ptr();
    p.u_batch_stride = u.stride(0); p.u_d_stride = u.stride(1);
    p.delta_batch_stride = delta.stride(0); p.delta_d_stride = delta.stride(1);
    p.A_d_stride = A.stride(0); p.A_dstate_stride = A.stride(1);
    p.B_batch_stride = B.stride(0); p.B_group_stride = B.stride(1); p.B_dstate_stride = B.stride(2);
    p.C_batch_stride = C.stride(0); p.C_group_stride = C.stride(1); p.C_dstate_stride = C.stride(2);
    p.out_batch_stride = out.stride(0); p.out_d_stride = out.stride(1);

    // Otherwise the kernel would be launched on device 0.  PyTorch-ROCm presents HIP devices under the "cuda"
    // device type, so the guard and the stream getter are the ones that understand that naming.
    const c10::hip::HIPGuardMasqueradingAsCUDA device_guard(u.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    const int rc = ss2d_selective_scan_fwd(&p, (void *)stream);
    TORCH_CHECK(rc == SS2D_OK, "ss2d_selective_scan_fwd: ", ss2d_strerror(rc), " (status ", rc, ")");
    return {out, x};
}

static std::vector<at::Tensor> selective_scan_bwd(const at::Tensor &u, const at::Tensor &delta, const at::Tensor &A,
                                                  const at::Tensor &B, const at::Tensor &C,
                                                  const c10::optional<at::Tensor> &D_,
                                                  const c10::optional<at::Tensor> &delta_bias_, const at::Tensor &dout,
                                                  const c10::optional<at::Tensor> &x_, bool delta_softplus, int nrows) {
    (void)nrows; (void)x_;   // the kernel recomputes the states it needs; the chunk states of the forward are unused
    const auto input_type = u.scalar_type();
    TORCH_CHECK(dtype_code(input_type) >= 0, "selective_scan_bwd not implemented for input type '", toString(input_type), "'");
    TORCH_CHECK(A.scalar_type() == at::ScalarType::Float, "A must be float32");
    TORCH_CHECK(dout.scalar_type() == input_type || dout.scalar_type() == at::ScalarType::Float, "dout must be u's dtype or float32");
    TORCH_CHECK(delta.scalar_type() == input_type && B.scalar_type() == input_type && C.scalar_type() == input_type,
                "delta, B, C must have the dtype of u");
    TORCH_CHECK(u.is_cuda() && delta.is_cuda() && A.is_cuda() && B.is_cuda() && C.is_cuda() && dout.is_cuda(), "inputs must be GPU tensors");
    TORCH_CHECK(u.dim() == 3 && delta.dim() == 3 && A.dim() == 2 && B.dim() == 4 && C.dim() == 4 && dout.dim() == 3, "bad tensor ranks");
    TORCH_CHECK(u.stride(-1) == 1 || u.size(-1) == 1);
    TORCH_CHECK(delta.stride(-1) == 1 || delta.size(-1) == 1);
    TORCH_CHECK(dout.stride(-1) == 1 || dout.size(-1) == 1);
    const int batch_size = u.size(0), dim = u.size(1), seqlen = u.size(2);
    const int dstate = A.size(1), n_groups = B.size(1), delta_dim = delta.size(1);
    TORCH_CHECK(dim % n_groups == 0, "dims should be dividable by n_groups");
    TORCH_CHECK(dim % delta_dim == 0, "dims should be dividable by delta_dim");
    TORCH_CHECK(dstate <= 256, "selective_scan only supports state dimension <= 256");
    CHECK_SHAPE(u, batch_size, dim, seqlen);
    CHECK_SHAPE(delta, batch_size, delta_dim, seqlen);
    CHECK_SHAPE(A, dim, dstate);
    CHECK_SHAPE(B, batch_size, n_groups, dstate, seqlen);
    TORCH_CHECK(B.stride(-1) == 1 || B.size(-1) == 1);
    CHECK_SHAPE(C, batch_size, n_groups, dstate, seqlen);
    TORCH_CHECK(C.stride(-1) == 1 || C.size(-1) == 1);
    CHECK_SHAPE(dout, batch_size, dim, seqlen);
    at::Tensor D, delta_bias;
    if (D_.has_value()) {
        D = D_.value().contiguous();
        TORCH_CHECK(D.scalar_type() == at::ScalarType::Float && D.is_cuda());
        CHECK_SHAPE(D, dim);
    }
    if (delta_bias_.has_value()) {
        delta_bias = delta_bias_.value().contiguous();
        TORCH_CHECK(delta_bias.scalar_type() == at::ScalarType::Float && delta_bias.is_cuda());
        CHECK_SHAPE(delta_bias, delta_dim);
    }

    const auto f32 = u.options().dtype(at::ScalarType::Float);
    at::Tensor du = torch::empty({batch_size, dim, seqlen}, u.options());
    at::Tensor ddelta = torch::empty({batch_size, dim, seqlen}, u.options());
    at::Tensor dA = torch::zeros({dim, dstate}, f32);
    at::Tensor dB = torch::zeros({batch_size, n_groups, dstate, seqlen}, f32);
    at::Tensor dC = torch::zeros({batch_size, n_groups, dstate, seqlen}, f32);
    at::Tensor dD, ddelta_bias;
    if (D.defined()) dD = torch::zeros({dim}, f32);
    if (delta_bias.defined()) ddelta_bias = torch::zeros({dim}, f32);

    ss2d_scan_bwd_params p = {};
    p.batch = batch_size; p.dim = dim; p.seqlen = seqlen; p.dstate = dstate; p.n_groups = n_groups; p.delta_dim = delta_dim;
    p.in_dtype = dtype_code(input_type);
    p.dout_dtype = dtype_code(dout.scalar_type());
    p.delta_softplus = delta_softplus ? 1 : 0;
    p.u = u.data_ptr(); p.delta = delta.data_ptr(); p.A = A.data_ptr(); p.B = B.data_ptr(); p.C = C.data_ptr();
    p.D = D.defined() ? D.data_ptr() : nullptr;
    p.delta_bias = delta_bias.defined() ? delta_bias.data_ptr() : nullptr;
    p.dout = dout.data_ptr();
    p.du = du.data_ptr(); p.ddelta = ddelta.data_ptr(); p.dA = dA.data_ptr(); p.dB = dB.data_ptr(); p.dC = dC.data_ptr();
    p.dD = dD.defined() ? dD.data_ptr() : nullptr;
    p.ddelta_bias = ddelta_bias.defined() ? ddelta_bias.data_ptr() : nullptr;
    p.u_batch_stride = u.stride(0); p.u_d_stride = u.stride(1);
    p.delta_batch_stride = delta.stride(0); p.delta_d_stride = delta.stride(1);
    p.A_d_stride = A.stride(0); p.A_dstate_stride = A.stride(1);
    p.B_batch_stride = B.stride(0); p.B_group_stride = B.stride(1); p.B_dstate_stride = B.stride(2);
    p.C_batch_stride = C.stride(0); p.C_group_stride = C.stride(1); p.C_dstate_stride = C.stride(2);
    p.dout_batch_stride = dout.stride(0); p.dout_d_stride = dout.stride(1);

    const c10::hip::HIPGuardMasqueradingAsCUDA device_guard(u.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    const int rc = ss2d_selective_scan_bwd(&p, (void *)stream);
    TORCH_CHECK(rc == SS2D_OK, "ss2d_selective_scan_bwd: ", ss2d_strerror(rc), " (status ", rc, ")");

    std::vector<at::Tensor> result = {du, ddelta, dA, dB.to(B.scalar_type()), dC.to(C.scalar_type()), dD, ddelta_bias};
    if (dim != delta_dim) {
        const int repeat = dim / delta_dim;
        result[1] = ddelta.view({batch_size, delta_dim, repeat, seqlen}).sum(2);
        if (ddelta_bias.defined()) result[6] = ddelta_bias.view({delta_dim, repeat}).sum(1);
    }
    return result;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "MI355X-native selective-scan forward behind the reference's extension interface";
    m.def("fwd", &selective_scan_fwd, "Selective scan forward (HIP, gfx950)");
    m.def("bwd", &selective_scan_bwd, "Selective scan backward (HIP, gfx950)");
}
