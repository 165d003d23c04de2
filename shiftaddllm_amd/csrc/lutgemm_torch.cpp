// Python module `lutgemm`: the reference extension's call signatures
// (lut_gemm/lutgemm_cuda.cpp:43-98,225-230 in the ShiftAddLLM checkout) on top
// of the gfx950 C ABI in lutgemm_gfx950.h.  Host-only translation unit: it
// validates tensors, picks the current HIP stream and forwards raw pointers.
//
// Differences from the reference bindings, all on the strict side:
//  * every operand is checked (dtype, device, contiguity, element counts) and a
//    violation raises instead of reading out of bounds;
//  * launches go to PyTorch's current stream of the output's device, not the
//    legacy default stream;
//  * `d_input` may hold M rows ([M, K] or [..., K]); the reference's row-wise
//    and uniform entry points are batch-1 only.
#include <torch/extension.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <string>

#include "lutgemm_gfx950.h"

namespace {

void check_common(const torch::Tensor &output, const torch::Tensor &bWeight,
                  const torch::Tensor &d_input, int64_t mSize, int64_t kSize, int64_t nb)
{
    TORCH_CHECK(output.is_cuda(), "output must be a GPU tensor");
    TORCH_CHECK(bWeight.is_cuda() && d_input.is_cuda(), "bWeight and d_input must be GPU tensors");
    TORCH_CHECK(bWeight.get_device() == output.get_device() &&
                    d_input.get_device() == output.get_device(),
                "all operands must live on the same device");
    TORCH_CHECK(output.scalar_type() == torch::kHalf, "output must be float16");
    TORCH_CHECK(d_input.scalar_type() == torch::kHalf, "d_input must be float16");
    TORCH_CHECK(bWeight.scalar_type() == torch::kInt32, "bWeight must be int32");
    TORCH_CHECK(output.is_contiguous() && bWeight.is_contiguous() && d_input.is_contiguous(),
                "operands must be contiguous");
    TORCH_CHECK(kSize > 0 && kSize % 32 == 0, "kSize must be a positive multiple of 32, got ", kSize);
    TORCH_CHECK(mSize > 0 && mSize % 4 == 0, "mSize must be a positive multiple of 4, got ", mSize);
    TORCH_CHECK(nb >= 1 && nb <= 4, "nb must be in 1..4, got ", nb);
    TORCH_CHECK(bWeight.numel() == (kSize / 32) * nb * mSize, "bWeight must hold [kSize/32, nb, mSize] = ",
                (kSize / 32) * nb * mSize, " words, got ", bWeight.numel());
    TORCH_CHECK(d_input.numel() > 0 && d_input.numel() % kSize == 0 && d_input.size(-1) == kSize,
                "d_input must be [..., kSize]");
    const int64_t rows = d_input.numel() / kSize;
    TORCH_CHECK(output.numel() == rows * mSize, "output must hold ", rows * mSize,
                " elements ([rows, mSize]), got ", output.numel());
}

void check_alpha(const torch::Tensor &alpha, const torch::Tensor &output, c10::ScalarType dtype,
                 int64_t numel, const char *what)
{
    TORCH_CHECK(alpha.is_cuda() && alpha.get_device() == output.get_device(), what,
                " must be on the output's device");
    TORCH_CHECK(alpha.scalar_type() == dtype, what, " has the wrong dtype: expected ",
                c10::toString(dtype), ", got ", c10::toString(alpha.scalar_type()));
    TORCH_CHECK(alpha.is_contiguous(), what, " must be contiguous");
    TORCH_CHECK(alpha.numel() == numel, what, " must hold ", numel, " elements, got ", alpha.numel());
}

void raise_on_error(int rc, const char *fn)
{
    if (rc == LUTGEMM_OK) return;
    std::string msg = std::string(fn) + ": " + lutgemm_strerror(rc);
    if (rc == LUTGEMM_EHIP || rc == LUTGEMM_ENOMEM)
        msg += " [hipError " + std::to_string(lutgemm_last_hip_error()) + "]";
    TORCH_CHECK(false, msg);
}

int rows_of(const torch::Tensor &d_input, int64_t kSize) { return (int)(d_input.numel() / kSize); }

}  // namespace

// lutgemm_cuda.cpp:43-52
void lutgemm_compute_shift_scale(torch::Tensor output, torch::Tensor bWeight, torch::Tensor alpha,
                                 torch::Tensor d_input, int64_t mSize, int64_t kSize, int64_t nb,
                                 int64_t num_groups)
{
    check_common(output, bWeight, d_input, mSize, kSize, nb);
    TORCH_CHECK(num_groups > 0 && kSize % num_groups == 0 && (kSize / num_groups) % 32 == 0,
                "kSize/num_groups must be a multiple of 32");
    check_alpha(alpha, output, torch::kHalf, num_groups * nb * mSize, "alpha [num_groups, nb, mSize]");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(output.device());
    int rc = lutgemm_gemv_rowwise_f16((const uint32_t *)bWeight.data_ptr<int32_t>(), alpha.data_ptr(),
                                      d_input.data_ptr(), output.data_ptr(), (int)mSize, (int)kSize,
                                      (int)nb, (int)num_groups, rows_of(d_input, kSize),
                                      c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
    raise_on_error(rc, "lutgemm_compute_shift_scale");
}

// lutgemm_cuda.cpp:88-98
void lutgemm_compute(torch::Tensor output, torch::Tensor bWeight, torch::Tensor alpha,
                     torch::Tensor q_bias, torch::Tensor d_input, int64_t mSize, int64_t kSize,
                     int64_t nb, int64_t num_groups)
{
    check_common(output, bWeight, d_input, mSize, kSize, nb);
    TORCH_CHECK(num_groups > 0 && kSize % num_groups == 0 && (kSize / num_groups) % 32 == 0,
                "kSize/num_groups must be a multiple of 32");
    check_alpha(alpha, output, torch::kHalf, num_groups * mSize, "alpha [num_groups, mSize]");
    check_alpha(q_bias, output, torch::kHalf, num_groups * mSize, "q_bias [num_groups, mSize]");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(output.device());
    int rc = lutgemm_gemv_uniform_f16((const uint32_t *)bWeight.data_ptr<int32_t>(), alpha.data_ptr(),
                                      q_bias.data_ptr(), d_input.data_ptr(), output.data_ptr(),
                                      (int)mSize, (int)kSize, (int)nb, (int)num_groups,
                                      rows_of(d_input, kSize),
                                      c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
    raise_on_error(rc, "lutgemm_compute");
}

static void check_block(int64_t mSize, int64_t num_groups)
{
    TORCH_CHECK(num_groups > 0 && mSize % num_groups == 0 && (mSize / num_groups) % 4 == 0,
                "mSize/num_groups (rows per alpha block) must be a multiple of 4");
}

// lutgemm_cuda.cpp:54-63
void lutgemm_compute_block(torch::Tensor output, torch::Tensor bWeight, torch::Tensor alpha,
                           torch::Tensor d_input, int64_t mSize, int64_t kSize, int64_t nb,
                           int64_t num_groups)
{
    check_common(output, bWeight, d_input, mSize, kSize, nb);
    check_block(mSize, num_groups);
    check_alpha(alpha, output, torch::kHalf, (kSize / 8) * nb * num_groups,
                "alpha [kSize/8, nb, num_groups]");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(output.device());
    int rc = lutgemm_gemv_block_f16((const uint32_t *)bWeight.data_ptr<int32_t>(), alpha.data_ptr(),
                                    d_input.data_ptr(), output.data_ptr(), (int)mSize, (int)kSize,
                                    (int)nb, (int)num_groups, rows_of(d_input, kSize),
                                    c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
    raise_on_error(rc, "lutgemm_compute_block");
}

// lutgemm_cuda.cpp:65-74
void lutgemm_compute_block_shift(torch::Tensor output, torch::Tensor bWeight, torch::Tensor alpha,
                                 torch::Tensor d_input, int64_t mSize, int64_t kSize, int64_t nb,
                                 int64_t num_groups, int64_t num_apot)
{
    check_common(output, bWeight, d_input, mSize, kSize, nb);
    check_block(mSize, num_groups);
    TORCH_CHECK(num_apot == 3, "num_apot must be 3 (the packed uint16 always carries three shift fields)");
    check_alpha(alpha, output, torch::kShort, (kSize / 8) * nb * num_groups,
                "alpha [kSize/8, nb, num_groups] (int16 holding uint16 shift fields)");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(output.device());
    int rc = lutgemm_gemv_block_shift_u16((const uint32_t *)bWeight.data_ptr<int32_t>(),
                                          (const uint16_t *)alpha.data_ptr<int16_t>(),
                                          d_input.data_ptr(), output.data_ptr(), (int)mSize,
                                          (int)kSize, (int)nb, (int)num_groups, (int)num_apot,
                                          rows_of(d_input, kSize),
                                          c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
    raise_on_error(rc, "lutgemm_compute_block_shift");
}

// lutgemm_cuda.cpp:76-85
void lutgemm_compute_block_shiftInt8(torch::Tensor output, torch::Tensor bWeight,
                                     torch::Tensor alpha, torch::Tensor d_input, int64_t mSize,
                                     int64_t kSize, int64_t nb, int64_t num_groups, int64_t num_apot)
{
    check_common(output, bWeight, d_input, mSize, kSize, nb);
    check_block(mSize, num_groups);
    TORCH_CHECK(num_apot == 3, "num_apot must be 3 (alpha carries three int8 exponents per entry)");
    check_alpha(alpha, output, torch::kChar, (kSize / 8) * nb * num_groups * 3,
                "alpha [kSize/8, nb, num_groups, 3]");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(output.device());
    int rc = lutgemm_gemv_block_apot_i8((const uint32_t *)bWeight.data_ptr<int32_t>(),
                                        alpha.data_ptr<int8_t>(), d_input.data_ptr(),
                                        output.data_ptr(), (int)mSize, (int)kSize, (int)nb,
                                        (int)num_groups, (int)num_apot, rows_of(d_input, kSize),
                                        c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
    raise_on_error(rc, "lutgemm_compute_block_shiftInt8");
}

// Calibration copy for profiler byte counters (no reference counterpart).
void copy_bytes(torch::Tensor dst, torch::Tensor src)
{
    TORCH_CHECK(dst.is_cuda() && src.is_cuda() && dst.is_contiguous() && src.is_contiguous(),
                "copy_bytes needs contiguous GPU tensors");
    TORCH_CHECK(dst.nbytes() == src.nbytes() && dst.nbytes() % 16 == 0, "sizes must match, multiple of 16");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(dst.device());
    int rc = lutgemm_copy_bytes(dst.data_ptr(), src.data_ptr(), dst.nbytes(),
                                c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
    raise_on_error(rc, "copy_bytes");
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.doc() = "MI355X (gfx950) LUT-GEMM engine behind the ShiftAddLLM `lutgemm` call signatures";
    m.def("lutgemm_compute", &lutgemm_compute, "uniform-quant LUT-GEMV (alpha, q_bias)");
    m.def("lutgemm_compute_shift_scale", &lutgemm_compute_shift_scale, "row-wise alpha LUT-GEMV");
    m.def("lutgemm_compute_block", &lutgemm_compute_block, "block alpha LUT-GEMV (fp16 alpha)");
    m.def("lutgemm_compute_block_shift", &lutgemm_compute_block_shift,
          "block alpha LUT-GEMV (uint16 shift fields)");
    m.def("lutgemm_compute_block_shiftInt8", &lutgemm_compute_block_shiftInt8,
          "block alpha LUT-GEMV (int8 exponents)");
    m.def("copy_bytes", &copy_bytes, "calibration copy kernel");
}
