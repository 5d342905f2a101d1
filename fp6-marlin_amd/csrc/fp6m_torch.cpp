// Thin PyTorch-ROCm extension: unwraps tensors, takes the current HIP stream and calls the C ABI of
// include/fp6m.h.  Module functions keep the names and argument order of the reference's two extensions
// (fp6_marlin/fp6_marlin_cuda.cpp:47-58,125-127: `mul`; fp6_marlin/pybind.cpp:89-94: `quantization_cpu`,
// `prepacking_cpu`, `dequantization_cpu`).  Errors surface as the reference's do: RuntimeError from `mul`
// (AT_ERROR), ValueError (std::invalid_argument) from the CPU routines.
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <stdexcept>
#include <string>

#include "fp6m.h"

namespace {

void check_cpu(int code)
{
    if (code != FP6M_OK) throw std::invalid_argument(fp6m_strerror(code));
}

void mul(const torch::Tensor& A, const torch::Tensor& B, torch::Tensor& C, const torch::Tensor& s,
         torch::Tensor& workspace, int quant_cols, int thread_k, int thread_n, int sms, int max_par, int group_size)
{
    TORCH_CHECK(A.is_cuda() && B.is_cuda() && C.is_cuda() && s.is_cuda() && workspace.is_cuda(),
                "all operands must be tensors on the GPU");
    TORCH_CHECK(A.is_contiguous() && B.is_contiguous() && C.is_contiguous() && s.is_contiguous() &&
                workspace.is_contiguous(), "all operands must be contiguous");
    TORCH_CHECK(A.scalar_type() == torch::kFloat16 && C.scalar_type() == torch::kFloat16 &&
                s.scalar_type() == torch::kFloat16, "A, C and s must be float16");
    TORCH_CHECK(B.element_size() == 4 && workspace.element_size() == 4, "B and workspace must hold 4-byte elements");
    TORCH_CHECK(A.dim() == 2 && C.dim() == 2 && C.size(0) == A.size(0), "A must be [m, k] and C [m, n]");
    const int dev = A.get_device();
    TORCH_CHECK(B.get_device() == dev && C.get_device() == dev && s.get_device() == dev && workspace.get_device() == dev,
                "all operands must live on the same device");
    const int prob_m = A.size(0), prob_n = C.size(1), prob_k = A.size(1);
    TORCH_CHECK(workspace.numel() >= prob_n / 128 * max_par, "workspace must be of size at least ",
                prob_n / 128 * max_par, ".");
    const int64_t qc = quant_cols <= 0 ? 0 : quant_cols, n4 = prob_n - qc;
    if (prob_k % 32 == 0 && qc <= prob_n) {
        const int64_t need_b = (int64_t)prob_k * n4 / 8 + (int64_t)prob_k * qc * 3 / 16;
        const int64_t need_s = (group_size == -1 ? n4 : (int64_t)(prob_k / 128) * n4) + qc;
        TORCH_CHECK(B.numel() >= need_b && s.numel() == need_s, "B must hold ", need_b, " words and s ", need_s,
                    " scales for this problem");
    }
    hipStream_t stream = c10::hip::getCurrentHIPStream(dev).stream();
    const int err = fp6m_mul(A.data_ptr(), B.data_ptr(), C.data_ptr(), s.data_ptr(), prob_m, prob_n, prob_k,
                             workspace.data_ptr(), dev, stream, thread_k, thread_n, sms, max_par, quant_cols, group_size);
    if (err == FP6M_ERR_PROB_SHAPE) {
        AT_ERROR("Problem (m=", prob_m, ", n=", prob_n, ", k=", prob_k, ")", " not compatible with thread_k=",
                 thread_k, ", thread_n=", thread_n, ".");
    } else if (err == FP6M_ERR_KERN_SHAPE) {
        AT_ERROR("No kernel implementation for thread_k=", thread_k, ", thread_n=", thread_n, ".");
    } else if (err != FP6M_OK) {
        AT_ERROR("fp6m_mul: ", fp6m_strerror(err), " (hip error ", fp6m_last_hip_error(), ")");
    }
}

torch::Tensor quantization_cpu(torch::Tensor w)
{
    if (w.scalar_type() != torch::kFloat16) throw std::invalid_argument("Input tensor should be of type float16.");
    if (w.is_cuda() || w.dim() != 2 || w.size(0) % 256 || w.size(1) % 256)
        throw std::invalid_argument("quantize expects a 2-D CPU tensor with both dimensions multiples of 256");
    w = w.contiguous();
    const int64_t oc = w.size(0), ic = w.size(1);
    auto out = torch::empty({ic, oc / 16 * 3}, torch::kInt32);
    // the flat buffer is read as ic rows of oc values, like the reference (pybind.cpp:52-57)
    check_cpu(fp6m_fp6_quantize(reinterpret_cast<const uint16_t*>(w.data_ptr()),
                                reinterpret_cast<uint8_t*>(out.data_ptr()), (size_t)ic, (size_t)oc));
    return out;
}

torch::Tensor prepacking_cpu(torch::Tensor q)
{
    if (q.scalar_type() != torch::kInt32 || q.is_cuda() || q.dim() != 2 || q.size(1) % 3)
        throw std::invalid_argument("prepacking expects a CPU int32 tensor [OC, IC*3/16]");
    q = q.contiguous();
    const int64_t oc = q.size(0), ic = q.size(1) * 16 / 3;
    if (oc % 256 || ic % 256) throw std::invalid_argument("prepacking expects OC and IC to be multiples of 256");
    auto out = torch::empty({ic / 32 * 3, oc * 2}, torch::kInt32);
    check_cpu(fp6m_fp6_prepack(out.data_ptr<int32_t>(), q.data_ptr<int32_t>(), (size_t)oc, (size_t)ic));
    return out;
}

torch::Tensor dequantization_cpu(torch::Tensor q, torch::Tensor scale)
{
    if (q.scalar_type() != torch::kInt32 || scale.scalar_type() != torch::kFloat16 || q.is_cuda() || scale.is_cuda() ||
        q.dim() != 2 || q.size(1) % 3 || scale.numel() != q.size(0))
        throw std::invalid_argument("dequantize expects CPU int32 [OC, IC*3/16] and float16 [OC]");
    q = q.contiguous();
    scale = scale.contiguous();
    const int64_t oc = q.size(0), ic = q.size(1) / 3 * 16;
    auto out = torch::empty({oc, ic}, torch::kFloat16);
    check_cpu(fp6m_fp6_dequant(reinterpret_cast<uint16_t*>(out.data_ptr()), reinterpret_cast<const uint8_t*>(q.data_ptr()),
                               (size_t)oc, (size_t)ic, reinterpret_cast<const uint16_t*>(scale.data_ptr())));
    return out;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    namespace py = pybind11;
    m.def("mul", &mul, "mixed INT4/FP6 x FP16 GEMM (gfx950)", py::arg("A"), py::arg("B"), py::arg("C"), py::arg("s"),
          py::arg("workspace"), py::arg("quant_cols") = -1, py::arg("thread_k") = -1, py::arg("thread_n") = -1,
          py::arg("sms") = -1, py::arg("max_par") = 8, py::arg("group_size") = -1);
    m.def("quantization_cpu", &quantization_cpu, "Weight quantization (CPU)");
    m.def("prepacking_cpu", &prepacking_cpu, "Weight prepacking (CPU)");
    m.def("dequantization_cpu", &dequantization_cpu, "Weight dequantization (CPU)");
}
