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
#include <vector>

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

// lutgemm_compute_shift_scale for alphas the caller knows to be powers of two (what the
// reference's quantiser produces, quantizers/bcq_quant/bcq_shift.py:15-24): a few rows on a large
// matrix take the block-scaled matrix-core kernel.  No counterpart in the reference's extension.
void lutgemm_compute_shift_scale_pow2(torch::Tensor output, torch::Tensor bWeight, torch::Tensor alpha,
                                      torch::Tensor d_input, int64_t mSize, int64_t kSize, int64_t nb,
                                      int64_t num_groups)
{
    check_common(output, bWeight, d_input, mSize, kSize, nb);
    TORCH_CHECK(num_groups > 0 && kSize % num_groups == 0 && (kSize / num_groups) % 32 == 0,
                "kSize/num_groups must be a multiple of 32");
    check_alpha(alpha, output, torch::kHalf, num_groups * nb * mSize, "alpha [num_groups, nb, mSize]");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(output.device());
    int rc = lutgemm_gemv_rowwise_pow2_f16((const uint32_t *)bWeight.data_ptr<int32_t>(), alpha.data_ptr(),
                                           d_input.data_ptr(), output.data_ptr(), (int)mSize, (int)kSize,
                                           (int)nb, (int)num_groups, rows_of(d_input, kSize),
                                           c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
    raise_on_error(rc, "lutgemm_compute_shift_scale_pow2");
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

// ---- test-data helpers of the reference module -------------------------------------
// (lut_gemm/lutgemm_cuda.cpp:104-223: makeRandom* fill a caller's tensor in place,
// element by element through index_put_; parsing moves host tensors to a device as the
// flat buffers the kernels read.)  Same signatures, the same value distributions and
// the same in-place contract, but generated by tensor operations on the tensor's own
// device, from PyTorch's generator of that device instead of the C library's rand().

// The reference's rand_fp32(): a random sign times the product of two uniforms in [0, 1].
torch::Tensor rand_fp32_like(const torch::Tensor &t, at::IntArrayRef shape)
{
    const auto opt = torch::TensorOptions().dtype(torch::kFloat32).device(t.device());
    const torch::Tensor sign = torch::randint(0, 2, shape, opt) * 2.0 - 1.0;
    return sign * torch::rand(shape, opt) * torch::rand(shape, opt);
}

void makeRandomInput(torch::Tensor inp, int64_t M, int64_t K)
{
    TORCH_CHECK(inp.dim() == 2 && inp.size(0) >= M && inp.size(1) >= K, "inp must be at least [M, K]");
    using namespace torch::indexing;
    inp.index_put_({Slice(0, M), Slice(0, K)}, rand_fp32_like(inp, {M, K}).to(inp.scalar_type()));
}

void makeRandomWeight(torch::Tensor qW, torch::Tensor bW, int64_t N, int64_t NUM_BITS, int64_t K)
{
    TORCH_CHECK(K % 32 == 0, "K must be a multiple of 32");
    TORCH_CHECK(qW.dim() == 3 && qW.size(0) >= K && qW.size(1) >= NUM_BITS && qW.size(2) >= N,
                "qW must be at least [K, NUM_BITS, N]");
    TORCH_CHECK(bW.dim() == 3 && bW.size(0) >= K / 32 && bW.size(1) >= NUM_BITS && bW.size(2) >= N,
                "bW must be at least [K/32, NUM_BITS, N]");
    TORCH_CHECK(bW.scalar_type() == torch::kInt32, "bW must be int32");
    using namespace torch::indexing;
    const auto opt = torch::TensorOptions().dtype(torch::kInt64).device(qW.device());
    const torch::Tensor bits = torch::randint(0, 2, {K, NUM_BITS, N}, opt);           // 1 <=> +1
    qW.index_put_({Slice(0, K), Slice(0, NUM_BITS), Slice(0, N)}, (bits * 2 - 1).to(qW.scalar_type()));
    // bit t of word k/32 <=> qW[k + t] = +1; the sum wraps bit 31 into the int32 sign
    const torch::Tensor weight = torch::ones({}, opt).bitwise_left_shift(torch::arange(32, opt)).view({1, 32, 1, 1});
    const torch::Tensor words = (bits.view({K / 32, 32, NUM_BITS, N}) * weight).sum(1);
    bW.index_put_({Slice(0, K / 32), Slice(0, NUM_BITS), Slice(0, N)}, words.to(torch::kInt32).to(bW.device()));
}

void makeRandomWeight_int3(torch::Tensor weight_int3, int64_t N, int64_t K_new)
{
    TORCH_CHECK(weight_int3.dim() == 2 && weight_int3.size(0) >= K_new && weight_int3.size(1) >= N,
                "weight_int3 must be at least [K_new, N]");
    using namespace torch::indexing;
    const auto opt = torch::TensorOptions().dtype(torch::kInt64).device(weight_int3.device());
    // rand(): uniform in [0, RAND_MAX]
    weight_int3.index_put_({Slice(0, K_new), Slice(0, N)},
                           torch::randint(0, (int64_t)2147483647, {K_new, N}, opt).to(weight_int3.scalar_type()));
}

void makeRandomAlpha(torch::Tensor alpha, torch::Tensor q_bias, int64_t num_groups, int64_t NUM_BITS, int64_t N)
{
    TORCH_CHECK(alpha.dim() == 3 && alpha.size(0) >= num_groups && alpha.size(1) >= NUM_BITS && alpha.size(2) >= N,
                "alpha must be at least [num_groups, NUM_BITS, N]");
    TORCH_CHECK(q_bias.dim() == 2 && q_bias.size(0) >= num_groups && q_bias.size(1) >= N,
                "q_bias must be at least [num_groups, N]");
    using namespace torch::indexing;
    q_bias.index_put_({Slice(0, num_groups), Slice(0, N)},
                      (rand_fp32_like(q_bias, {num_groups, N}) / (double)(1 << NUM_BITS)).to(q_bias.scalar_type()));
    const auto opt = torch::TensorOptions().dtype(torch::kFloat32).device(alpha.device());
    const torch::Tensor scale = torch::exp2(-torch::arange(NUM_BITS, opt)).view({1, NUM_BITS, 1});   // 1 / 2^b
    alpha.index_put_({Slice(0, num_groups), Slice(0, NUM_BITS), Slice(0, N)},
                     (rand_fp32_like(alpha, {num_groups, NUM_BITS, N}) * scale).to(alpha.scalar_type()));
}

void makeRandomScale(torch::Tensor scale, int64_t N)
{
    TORCH_CHECK(scale.dim() == 1 && scale.size(0) >= N, "scale must hold at least N elements");
    using namespace torch::indexing;
    scale.index_put_({Slice(0, N)}, rand_fp32_like(scale, {N}).to(scale.scalar_type()));
}

void makeRandomBias(torch::Tensor bias, int64_t N) { makeRandomScale(bias, N); }

// bW int32 (any shape, kSize * mSize * nb / 32 words), A and q_bias floating point with
// at least num_groups * mSize * nb and num_groups * mSize elements -> flat device
// tensors {bWeight int32, q_bias fp16, alpha fp16} on GPU `cuda`
// (lut_gemm/lutgemm_cuda.cpp:173-223).
std::vector<torch::Tensor> parsing(torch::Tensor bW, torch::Tensor A, int64_t row, int64_t col, int64_t num_bits,
                                   bool is_row_wise_quantize, int64_t num_alpha_groups, torch::Tensor q_bias,
                                   int64_t cuda)
{
    const int64_t mSize = is_row_wise_quantize ? row : col, kSize = is_row_wise_quantize ? col : row;
    const int64_t words = kSize * mSize * num_bits / 32;
    TORCH_CHECK(bW.scalar_type() == torch::kInt32 && bW.numel() >= words, "bW must hold ", words, " int32 words");
    TORCH_CHECK(A.numel() >= num_alpha_groups * mSize * num_bits, "A must hold num_groups * mSize * nb elements");
    TORCH_CHECK(q_bias.numel() >= num_alpha_groups * mSize, "q_bias must hold num_groups * mSize elements");
    const torch::Device dev(torch::kCUDA, (c10::DeviceIndex)cuda);
    const torch::Tensor p_q_bias = q_bias.reshape({-1}).narrow(0, 0, num_alpha_groups * mSize).to(dev, torch::kHalf);
    const torch::Tensor p_alpha = A.reshape({-1}).narrow(0, 0, num_alpha_groups * mSize * num_bits).to(dev, torch::kHalf);
    const torch::Tensor bWeight = bW.reshape({-1}).narrow(0, 0, words).to(dev).contiguous();
    return {bWeight, p_q_bias.contiguous(), p_alpha.contiguous()};
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.doc() = "MI355X (gfx950) LUT-GEMM engine behind the ShiftAddLLM `lutgemm` call signatures";
    m.def("lutgemm_compute", &lutgemm_compute, "uniform-quant LUT-GEMV (alpha, q_bias)");
    m.def("lutgemm_compute_shift_scale", &lutgemm_compute_shift_scale, "row-wise alpha LUT-GEMV");
    m.def("lutgemm_compute_shift_scale_pow2", &lutgemm_compute_shift_scale_pow2,
          "row-wise alpha LUT-GEMV, alphas promised to be powers of two");
    m.def("lutgemm_compute_block", &lutgemm_compute_block, "block alpha LUT-GEMV (fp16 alpha)");
    m.def("lutgemm_compute_block_shift", &lutgemm_compute_block_shift,
          "block alpha LUT-GEMV (uint16 shift fields)");
    m.def("lutgemm_compute_block_shiftInt8", &lutgemm_compute_block_shiftInt8,
          "block alpha LUT-GEMV (int8 exponents)");
    m.def("makeRandomInput", &makeRandomInput, "fill inp[:M, :K] with the reference's random activations");
    m.def("makeRandomAlpha", &makeRandomAlpha, "fill alpha [num_groups, NUM_BITS, N] and q_bias [num_groups, N]");
    m.def("makeRandomBias", &makeRandomBias, "fill bias[:N]");
    m.def("makeRandomScale", &makeRandomScale, "fill scale[:N]");
    m.def("makeRandomWeight_int3", &makeRandomWeight_int3, "fill weight_int3[:K_new, :N] with random words");
    m.def("makeRandomWeight", &makeRandomWeight, "fill qW [K, NUM_BITS, N] with +-1 and bW [K/32, NUM_BITS, N] with their packing");
    m.def("parsing", &parsing, "host tensors -> flat device buffers {bWeight, q_bias, alpha}");
    m.def("copy_bytes", &copy_bytes, "calibration copy kernel");
}
