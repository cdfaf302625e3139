// PyTorch-ROCm binding of the MACKO path: registers the `macko_spmv` operator library and
// forwards to the C ABI of libmacko_hip.so on torch's current HIP stream.
//
// Mirrors the upstream torch boundary:
//   macko_spmv::multiply  <- TORCH_LIBRARY block in src/macko_spmv/__init__.py:56-63 and
//                            macko_spmv_launcher, src/macko_spmv/cuda/kernels_torch_launchers.cuh:3-48
//   macko_spmv::compress  <- cpu_compress, src/macko_spmv/cuda/cpu_compressor_torch_launcher.cuh:6-39
// HIP tensors carry the "cuda" device type and dispatch on the CUDA key in PyTorch-ROCm, hence
// the *MasqueradingAsCUDA guard and stream accessors.  There is deliberately no CPU kernel
// for multiply: without a GPU the operator raises.

#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <chrono>
#include <tuple>

#include "macko_decode.h"
#include "macko_hip.h"

namespace {

void check_rc(int rc, const char *what)
{
    TORCH_CHECK(rc == 0, "macko_spmv: ", what, " failed: ", macko_hip_error_string(rc), " (code ", rc, ")");
}

// What every product operator checks about the compressed matrix (the upstream launcher checks the
// value dtype only, src/macko_spmv/cuda/kernels_torch_launchers.cuh:10-11; its data_ptr<T>() calls
// throw on the other two).
void check_macko_operands(const at::Tensor &M_values, const at::Tensor &M_deltas, const at::Tensor &M_row_indices,
                          int64_t M_rows, int64_t M_cols, at::ScalarType value_type = at::kHalf)
{
    TORCH_CHECK(M_values.dtype() == value_type, value_type == at::kHalf ? "M must be torch.half" : "M must be torch.int8");
    TORCH_CHECK(M_deltas.dtype() == at::kByte, "M_deltas must be torch.uint8");
    TORCH_CHECK(M_row_indices.dtype() == at::kInt, "M_row_indices must be torch.int32");
    TORCH_CHECK(M_values.is_cuda() && M_deltas.is_cuda() && M_row_indices.is_cuda(), "the matrix must live on the GPU");
    TORCH_CHECK(M_values.is_contiguous() && M_deltas.is_contiguous() && M_row_indices.is_contiguous(),
                "the matrix tensors must be contiguous");
    TORCH_CHECK(M_rows >= 0 && M_cols >= 0 && M_rows < (1ll << 31) && M_cols < (1ll << 31), "bad dimensions");
    TORCH_CHECK(M_row_indices.numel() >= M_rows + 1, "M_row_indices must hold M_rows + 1 elements");
    TORCH_CHECK(M_deltas.numel() * 2 >= M_values.numel(), "M_deltas must hold one nibble per value");
}

void check_half_gpu(const at::Tensor &t, const char *name)
{
    TORCH_CHECK(t.dtype() == at::kHalf, name, " must be torch.half");
    TORCH_CHECK(t.is_cuda() && t.is_contiguous(), name, " must be a contiguous GPU tensor");
}

at::Tensor multiply_hip(const at::Tensor &M_values, const at::Tensor &M_deltas, const at::Tensor &M_row_indices,
                        int64_t M_rows, int64_t M_cols, const at::Tensor &V)
{
    check_macko_operands(M_values, M_deltas, M_row_indices, M_rows, M_cols);
    check_half_gpu(V, "V");
    TORCH_CHECK(V.numel() >= M_cols || M_values.numel() == 0, "V must hold at least M_cols elements");

    const c10::hip::HIPGuardMasqueradingAsCUDA guard(M_values.device());
    at::Tensor C = at::empty({M_rows}, M_values.options());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    const int rc = macko_spmv_f16(M_values.data_ptr(), M_deltas.data_ptr(), M_row_indices.data_ptr<int>(),
                                  V.data_ptr(), C.data_ptr(), (int32_t)M_rows, (int32_t)M_cols,
                                  M_values.numel(), (void *)stream);
    check_rc(rc, "multiply");
    return C;
}

// Where every wave of the product's launch starts (macko_spmv_plan_build): int32 [entries], empty if
// products of this shape take none.  Built once per matrix, after compressing.
at::Tensor plan_hip(const at::Tensor &M_row_indices, int64_t M_rows, int64_t M_cols, int64_t padded_entries)
{
    TORCH_CHECK(M_row_indices.dtype() == at::kInt && M_row_indices.is_cuda() && M_row_indices.is_contiguous(),
                "M_row_indices must be a contiguous torch.int32 GPU tensor");
    TORCH_CHECK(M_rows >= 0 && M_cols >= 0 && M_rows < (1ll << 31) && M_cols < (1ll << 31), "bad dimensions");
    TORCH_CHECK(M_row_indices.numel() >= M_rows + 1, "M_row_indices must hold M_rows + 1 elements");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(M_row_indices.device());
    int32_t entries = 0;
    check_rc(macko_spmv_plan_entries((int32_t)M_rows, (int32_t)M_cols, padded_entries, &entries), "plan");
    at::Tensor plan = at::empty({entries}, M_row_indices.options());
    if (entries == 0) return plan;
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    check_rc(macko_spmv_plan_build(M_row_indices.data_ptr<int>(), (int32_t)M_rows, (int32_t)M_cols, padded_entries,
                                   plan.data_ptr<int>(), entries, (void *)stream),
             "plan");
    return plan;
}

void check_plan(const at::Tensor &plan, const at::Tensor &M_values)
{
    TORCH_CHECK(plan.dtype() == at::kInt && plan.is_contiguous(), "plan must be a contiguous torch.int32 tensor");
    TORCH_CHECK(plan.numel() == 0 || (plan.is_cuda() && plan.device() == M_values.device()),
                "plan must live on the matrix's GPU");
}

at::Tensor multiply_planned_hip(const at::Tensor &M_values, const at::Tensor &M_deltas,
                                const at::Tensor &M_row_indices, int64_t M_rows, int64_t M_cols, const at::Tensor &V,
                                const at::Tensor &plan)
{
    check_macko_operands(M_values, M_deltas, M_row_indices, M_rows, M_cols);
    check_half_gpu(V, "V");
    check_plan(plan, M_values);
    TORCH_CHECK(V.numel() >= M_cols || M_values.numel() == 0, "V must hold at least M_cols elements");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(M_values.device());
    at::Tensor C = at::empty({M_rows}, M_values.options());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    const int rc = macko_spmv_f16_planned(M_values.data_ptr(), M_deltas.data_ptr(), M_row_indices.data_ptr<int>(),
                                          plan.numel() ? plan.data_ptr<int>() : nullptr, (int32_t)plan.numel(),
                                          V.data_ptr(), C.data_ptr(), (int32_t)M_rows, (int32_t)M_cols,
                                          M_values.numel(), (void *)stream);
    check_rc(rc, "multiply_planned");
    return C;
}

void multiply_axpby_planned_hip(const at::Tensor &M_values, const at::Tensor &M_deltas,
                                const at::Tensor &M_row_indices, int64_t M_rows, int64_t M_cols, const at::Tensor &V,
                                at::Tensor C, double alpha, double beta, const at::Tensor &plan)
{
    check_macko_operands(M_values, M_deltas, M_row_indices, M_rows, M_cols);
    check_half_gpu(V, "V");
    check_half_gpu(C, "C");
    check_plan(plan, M_values);
    TORCH_CHECK(C.numel() >= M_rows, "C must hold M_rows elements");
    TORCH_CHECK(V.numel() >= M_cols || M_values.numel() == 0, "V must hold at least M_cols elements");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(M_values.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    const int rc = macko_spmv_f16_axpby_planned(
        M_values.data_ptr(), M_deltas.data_ptr(), M_row_indices.data_ptr<int>(),
        plan.numel() ? plan.data_ptr<int>() : nullptr, (int32_t)plan.numel(), V.data_ptr(), C.data_ptr(),
        (int32_t)M_rows, (int32_t)M_cols, M_values.numel(), (float)alpha, (float)beta, (void *)stream);
    check_rc(rc, "multiply_axpby_planned");
}

// Y[b] = M @ X[b] for X of shape [batch, M_cols] -> [batch, M_rows].
at::Tensor multiply_batched_hip(const at::Tensor &M_values, const at::Tensor &M_deltas,
                                const at::Tensor &M_row_indices, int64_t M_rows, int64_t M_cols, const at::Tensor &X)
{
    check_macko_operands(M_values, M_deltas, M_row_indices, M_rows, M_cols);
    check_half_gpu(X, "X");
    TORCH_CHECK(X.dim() == 2 && X.size(1) >= M_cols, "X must be [batch, >= M_cols]");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(M_values.device());
    at::Tensor Y = at::empty({X.size(0), M_rows}, M_values.options());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    check_rc(macko_spmv_f16_batched(M_values.data_ptr(), M_deltas.data_ptr(), M_row_indices.data_ptr<int>(),
                                    X.data_ptr(), Y.data_ptr(), (int32_t)M_rows, (int32_t)M_cols, M_values.numel(),
                                    (int32_t)X.size(0), X.size(1), M_rows, (void *)stream),
             "multiply_batched");
    return Y;
}

// C = alpha * (M @ V) + beta * C, in place on C.
void multiply_axpby_hip(const at::Tensor &M_values, const at::Tensor &M_deltas, const at::Tensor &M_row_indices,
                        int64_t M_rows, int64_t M_cols, const at::Tensor &V, at::Tensor C, double alpha,
                        double beta)
{
    check_macko_operands(M_values, M_deltas, M_row_indices, M_rows, M_cols);
    check_half_gpu(V, "V");
    check_half_gpu(C, "C");
    TORCH_CHECK(C.numel() >= M_rows, "C must hold M_rows elements");
    TORCH_CHECK(V.numel() >= M_cols || M_values.numel() == 0, "V must hold at least M_cols elements");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(M_values.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    const int rc = macko_spmv_f16_axpby(M_values.data_ptr(), M_deltas.data_ptr(), M_row_indices.data_ptr<int>(),
                                        V.data_ptr(), C.data_ptr(), (int32_t)M_rows, (int32_t)M_cols,
                                        M_values.numel(), (float)alpha, (float)beta, (void *)stream);
    check_rc(rc, "multiply_axpby");
}

std::tuple<at::Tensor, at::Tensor, at::Tensor, int64_t, int64_t> compress_on_device(const at::Tensor &M)
{
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(M.device());
    const int64_t rows = M.size(0), cols = M.size(1);
    TORCH_CHECK(rows * cols < (1ll << 31), "matrix too large: rows * cols must stay below 2^31");
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    {
        // The host has to wait for the entry count in the middle of this call, which a stream
        // that is being captured into a graph cannot give: say so instead of breaking the capture.
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        const hipError_t e = hipStreamIsCapturing(stream, &capturing);
        TORCH_CHECK(e == hipSuccess, "macko_spmv: compress: ", hipGetErrorString(e));
        TORCH_CHECK(capturing == hipStreamCaptureStatusNone,
                    "macko_spmv: compress cannot be captured into a HIP graph (the sizes of its outputs depend on "
                    "the data); compress outside the capture and capture multiply only");
    }
    const bool int8 = M.dtype() == at::kChar;
    at::Tensor row_ptr = at::empty({rows + 1}, M.options().dtype(at::kInt));
    // The entry count sizes the outputs, so the host has to wait for it.  The count pass stores it
    // into a page-locked word of this thread's, which the thread watches for a short while (a
    // matrix of a few thousand rows and columns is through in about ten microseconds, and the
    // store is seen much sooner than a stream synchronization returns); for anything longer it
    // falls back to waiting for the stream.
    // (never released: at thread or process exit the runtime it would go back to may be gone already)
    thread_local at::Tensor *total_word =
        new at::Tensor(at::empty({1}, at::TensorOptions().dtype(at::kInt).pinned_memory(true)));
    volatile int *total = total_word->data_ptr<int>();
    *total = -1;
    check_rc((int8 ? macko_compress_i8_count_total : macko_compress_f16_count_total)(
                 M.data_ptr(), (int32_t)rows, (int32_t)cols, row_ptr.data_ptr<int>(), total_word->data_ptr<int>(),
                 (void *)stream),
             "compress (count)");
    const auto give_up = std::chrono::steady_clock::now() + std::chrono::microseconds(200);
    while (__atomic_load_n(total, __ATOMIC_ACQUIRE) < 0 && std::chrono::steady_clock::now() < give_up) {
    }
    if (__atomic_load_n(total, __ATOMIC_ACQUIRE) < 0) {
        const hipError_t e = hipStreamSynchronize(stream);
        TORCH_CHECK(e == hipSuccess, "macko_spmv: compress (waiting for the entry count): ", hipGetErrorString(e));
    }
    const int64_t n = __atomic_load_n(total, __ATOMIC_ACQUIRE);
    TORCH_CHECK(n >= 0, "macko_spmv: compress: the count pass did not deliver the entry count");
    const int64_t padded = (n + 7) / 8 * 8;
    at::Tensor values = at::empty({padded}, M.options());
    at::Tensor deltas = at::empty({padded / 2}, M.options().dtype(at::kByte));
    check_rc((int8 ? macko_compress_i8_fill : macko_compress_f16_fill)(
                 M.data_ptr(), (int32_t)rows, (int32_t)cols, row_ptr.data_ptr<int>(), values.data_ptr(),
                 deltas.data_ptr(), padded, (void *)stream),
             "compress (fill)");
    return std::make_tuple(values, deltas, row_ptr, rows, cols);
}

// HIP tensor in -> HIP tensors out.
std::tuple<at::Tensor, at::Tensor, at::Tensor, int64_t, int64_t> compress_hip(const at::Tensor &M)
{
    TORCH_CHECK(M.dtype() == at::kHalf, "M must be torch.half");
    TORCH_CHECK(M.dim() == 2, "M must be a matrix");
    TORCH_CHECK(M.is_contiguous(), "M must be contiguous");
    return compress_on_device(M);
}

// CPU tensor in -> CPU tensors out, like the upstream cpu_compress, but the work is done by the
// HIP compressor: the matrix is staged to the current GPU and the three arrays are copied back.
// Needs a GPU; there is no host implementation.
std::tuple<at::Tensor, at::Tensor, at::Tensor, int64_t, int64_t> compress_cpu(const at::Tensor &M)
{
    TORCH_CHECK(M.dtype() == at::kHalf, "M must be torch.half");
    TORCH_CHECK(M.dim() == 2, "M must be a matrix");
    TORCH_CHECK(M.is_contiguous(), "M must be contiguous");
    int n_dev = 0;
    TORCH_CHECK(hipGetDeviceCount(&n_dev) == hipSuccess && n_dev > 0,
                "macko_spmv: compress needs an AMD GPU (the compressor is a HIP kernel; there is no CPU path)");
    auto out = compress_on_device(M.to(at::Device(at::kCUDA, c10::hip::current_device())));
    return std::make_tuple(std::get<0>(out).cpu(), std::get<1>(out).cpu(), std::get<2>(out).cpu(),
                           std::get<3>(out), std::get<4>(out));
}

// int8 twins (compress_rows_int8_cpu, src/macko_spmv/cuda/cpu_compressor.cuh:75-117, and
// macko_spmv_int8, src/macko_spmv/cuda/kernels.cuh:126-216; upstream exposes them only in its C
// benchmark, c_benchmarking/benchmark.cu:106-118).
std::tuple<at::Tensor, at::Tensor, at::Tensor, int64_t, int64_t> compress_int8_hip(const at::Tensor &M)
{
    TORCH_CHECK(M.dtype() == at::kChar, "M must be torch.int8");
    TORCH_CHECK(M.dim() == 2, "M must be a matrix");
    TORCH_CHECK(M.is_contiguous(), "M must be contiguous");
    return compress_on_device(M);
}

std::tuple<at::Tensor, at::Tensor, at::Tensor, int64_t, int64_t> compress_int8_cpu(const at::Tensor &M)
{
    TORCH_CHECK(M.dtype() == at::kChar, "M must be torch.int8");
    TORCH_CHECK(M.dim() == 2, "M must be a matrix");
    TORCH_CHECK(M.is_contiguous(), "M must be contiguous");
    int n_dev = 0;
    TORCH_CHECK(hipGetDeviceCount(&n_dev) == hipSuccess && n_dev > 0,
                "macko_spmv: compress needs an AMD GPU (the compressor is a HIP kernel; there is no CPU path)");
    auto out = compress_on_device(M.to(at::Device(at::kCUDA, c10::hip::current_device())));
    return std::make_tuple(std::get<0>(out).cpu(), std::get<1>(out).cpu(), std::get<2>(out).cpu(),
                           std::get<3>(out), std::get<4>(out));
}

void check_int8_operands(const at::Tensor &M_values, const at::Tensor &M_deltas, const at::Tensor &M_row_indices,
                         int64_t M_rows, int64_t M_cols, const at::Tensor &V)
{
    check_macko_operands(M_values, M_deltas, M_row_indices, M_rows, M_cols, at::kChar);
    check_half_gpu(V, "V");
    TORCH_CHECK(V.numel() >= M_cols || M_values.numel() == 0, "V must hold at least M_cols elements");
}

at::Tensor multiply_int8_hip(const at::Tensor &M_values, const at::Tensor &M_deltas,
                             const at::Tensor &M_row_indices, int64_t M_rows, int64_t M_cols, const at::Tensor &V)
{
    check_int8_operands(M_values, M_deltas, M_row_indices, M_rows, M_cols, V);
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(M_values.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    at::Tensor C = at::empty({M_rows}, V.options());
    check_rc(macko_spmv_i8f16(M_values.data_ptr(), M_deltas.data_ptr(), M_row_indices.data_ptr<int>(),
                              V.data_ptr(), C.data_ptr(), (int32_t)M_rows, (int32_t)M_cols, M_values.numel(),
                              (void *)stream),
             "multiply_int8");
    return C;
}

// C = alpha * (M @ V) + beta * C, in place on C.
void multiply_int8_axpby_hip(const at::Tensor &M_values, const at::Tensor &M_deltas,
                             const at::Tensor &M_row_indices, int64_t M_rows, int64_t M_cols, const at::Tensor &V,
                             at::Tensor C, double alpha, double beta)
{
    check_int8_operands(M_values, M_deltas, M_row_indices, M_rows, M_cols, V);
    TORCH_CHECK(C.dtype() == at::kHalf && C.is_cuda() && C.is_contiguous() && C.numel() >= M_rows,
                "C must be a contiguous torch.half GPU tensor with at least M_rows elements");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(M_values.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    check_rc(macko_spmv_i8f16_axpby(M_values.data_ptr(), M_deltas.data_ptr(), M_row_indices.data_ptr<int>(),
                                    V.data_ptr(), C.data_ptr(), (int32_t)M_rows, (int32_t)M_cols, M_values.numel(),
                                    (float)alpha, (float)beta, (void *)stream),
             "multiply_int8_axpby");
}

at::Tensor decompress_hip(const at::Tensor &M_values, const at::Tensor &M_deltas, const at::Tensor &M_row_indices,
                          int64_t M_rows, int64_t M_cols)
{
    check_macko_operands(M_values, M_deltas, M_row_indices, M_rows, M_cols);
    TORCH_CHECK(M_rows * M_cols < (1ll << 31), "matrix too large: rows * cols must stay below 2^31");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(M_values.device());
    at::Tensor dense = at::empty({M_rows, M_cols}, M_values.options());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    check_rc(macko_decompress_f16(M_values.data_ptr(), M_deltas.data_ptr(), M_row_indices.data_ptr<int>(),
                                  (int32_t)M_rows, (int32_t)M_cols, M_values.numel(), dense.data_ptr(), (void *)stream),
             "decompress");
    return dense;
}

// ---- glue kernels of the decode harness (include/macko_decode.h) -------------------------------

at::Tensor decode_rmsnorm_hip(const at::Tensor &x, const at::Tensor &weight, double eps)
{
    check_half_gpu(x, "x");
    check_half_gpu(weight, "weight");
    TORCH_CHECK(weight.numel() == x.numel(), "weight and x must have the same length");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    at::Tensor y = at::empty_like(x);
    check_rc(macko_decode_rmsnorm_f16(x.data_ptr(), weight.data_ptr(), y.data_ptr(), (int32_t)x.numel(), (float)eps,
                                      (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
             "decode_rmsnorm");
    return y;
}

// q, k, v: [n_heads * head_dim]; caches [n_heads, max_len, head_dim] (updated in place); returns rotated q.
at::Tensor decode_rope_append_hip(const at::Tensor &q, const at::Tensor &k, const at::Tensor &v,
                                  const at::Tensor &cos_table, const at::Tensor &sin_table,
                                  const at::Tensor &position, at::Tensor k_cache, at::Tensor v_cache)
{
    check_half_gpu(q, "q");
    check_half_gpu(k, "k");
    check_half_gpu(v, "v");
    check_half_gpu(k_cache, "k_cache");
    check_half_gpu(v_cache, "v_cache");
    TORCH_CHECK(k_cache.dim() == 3 && v_cache.sizes() == k_cache.sizes(), "caches must be [heads, max_len, head_dim]");
    const int64_t n_heads = k_cache.size(0), max_len = k_cache.size(1), head_dim = k_cache.size(2);
    TORCH_CHECK(q.numel() == n_heads * head_dim && k.numel() == q.numel() && v.numel() == q.numel(), "bad q/k/v size");
    TORCH_CHECK(cos_table.is_cuda() && cos_table.dtype() == at::kFloat && cos_table.is_contiguous() &&
                    cos_table.numel() == max_len * (head_dim / 2) && sin_table.is_cuda() &&
                    sin_table.dtype() == at::kFloat && sin_table.is_contiguous() &&
                    sin_table.numel() == cos_table.numel(),
                "cos/sin tables must be contiguous float32 GPU tensors [max_len, head_dim/2]");
    TORCH_CHECK(position.is_cuda() && position.dtype() == at::kLong && position.numel() == 1, "bad position");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
    at::Tensor q_out = at::empty_like(q);
    check_rc(macko_decode_rope_append_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), cos_table.data_ptr<float>(),
                                          sin_table.data_ptr<float>(), position.data_ptr<int64_t>(), q_out.data_ptr(),
                                          k_cache.data_ptr(), v_cache.data_ptr(), (int32_t)n_heads, (int32_t)head_dim,
                                          (int32_t)max_len,
                                          (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
             "decode_rope_append");
    return q_out;
}

at::Tensor decode_attention_hip(const at::Tensor &q, const at::Tensor &k_cache, const at::Tensor &v_cache,
                                const at::Tensor &position, double scale)
{
    check_half_gpu(q, "q");
    check_half_gpu(k_cache, "k_cache");
    check_half_gpu(v_cache, "v_cache");
    TORCH_CHECK(k_cache.dim() == 3 && v_cache.sizes() == k_cache.sizes(), "caches must be [heads, max_len, head_dim]");
    const int64_t n_heads = k_cache.size(0), max_len = k_cache.size(1), head_dim = k_cache.size(2);
    TORCH_CHECK(q.numel() == n_heads * head_dim, "bad q size");
    TORCH_CHECK(position.is_cuda() && position.dtype() == at::kLong && position.numel() == 1, "bad position");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
    at::Tensor out = at::empty_like(q);
    check_rc(macko_decode_attention_f16(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                        position.data_ptr<int64_t>(), out.data_ptr(), (int32_t)n_heads,
                                        (int32_t)head_dim, (int32_t)max_len, (float)scale,
                                        (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
             "decode_attention");
    return out;
}

at::Tensor decode_silu_mul_hip(const at::Tensor &gate, const at::Tensor &up)
{
    check_half_gpu(gate, "gate");
    check_half_gpu(up, "up");
    TORCH_CHECK(gate.numel() == up.numel(), "gate and up must have the same length");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(gate.device());
    at::Tensor out = at::empty_like(gate);
    check_rc(macko_decode_silu_mul_f16(gate.data_ptr(), up.data_ptr(), out.data_ptr(), (int32_t)gate.numel(),
                                       (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
             "decode_silu_mul");
    return out;
}

// M @ rmsnorm(V): the norm is applied while V is staged for the product.
at::Tensor multiply_rmsnorm_hip(const at::Tensor &M_values, const at::Tensor &M_deltas,
                                const at::Tensor &M_row_indices, int64_t M_rows, int64_t M_cols, const at::Tensor &V,
                                const at::Tensor &norm_weight, double eps)
{
    check_macko_operands(M_values, M_deltas, M_row_indices, M_rows, M_cols);
    check_half_gpu(V, "V");
    check_half_gpu(norm_weight, "norm_weight");
    TORCH_CHECK(V.numel() == M_cols && norm_weight.numel() == M_cols, "V and norm_weight must hold M_cols elements");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(M_values.device());
    at::Tensor C = at::empty({M_rows}, M_values.options());
    check_rc(macko_spmv_f16_rmsnorm(M_values.data_ptr(), M_deltas.data_ptr(), M_row_indices.data_ptr<int>(),
                                    V.data_ptr(), norm_weight.data_ptr(), (float)eps, C.data_ptr(), (int32_t)M_rows,
                                    (int32_t)M_cols, M_values.numel(),
                                    (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
             "multiply_rmsnorm");
    return C;
}

// C = alpha * M @ (silu(gate) * up) + beta * C, in place on C.
void multiply_silu_mul_axpby_hip(const at::Tensor &M_values, const at::Tensor &M_deltas,
                                 const at::Tensor &M_row_indices, int64_t M_rows, int64_t M_cols,
                                 const at::Tensor &gate, const at::Tensor &up, at::Tensor C, double alpha, double beta)
{
    check_macko_operands(M_values, M_deltas, M_row_indices, M_rows, M_cols);
    check_half_gpu(gate, "gate");
    check_half_gpu(up, "up");
    check_half_gpu(C, "C");
    TORCH_CHECK(gate.numel() == M_cols && up.numel() == M_cols, "gate and up must hold M_cols elements");
    TORCH_CHECK(C.numel() >= M_rows, "C must hold M_rows elements");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(M_values.device());
    check_rc(macko_spmv_f16_silu_mul_axpby(M_values.data_ptr(), M_deltas.data_ptr(), M_row_indices.data_ptr<int>(),
                                           gate.data_ptr(), up.data_ptr(), C.data_ptr(), (int32_t)M_rows,
                                           (int32_t)M_cols, M_values.numel(), (float)alpha, (float)beta,
                                           (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
             "multiply_silu_mul_axpby");
}

// Rotary embedding, cache append and attention of one decode step in one launch; q, k, v are the
// raw projections.  Returns the attention output [n_heads * head_dim].
at::Tensor decode_rope_attention_hip(const at::Tensor &q, const at::Tensor &k, const at::Tensor &v,
                                     const at::Tensor &cos_table, const at::Tensor &sin_table,
                                     const at::Tensor &position, at::Tensor k_cache, at::Tensor v_cache, double scale)
{
    check_half_gpu(q, "q");
    check_half_gpu(k, "k");
    check_half_gpu(v, "v");
    check_half_gpu(k_cache, "k_cache");
    check_half_gpu(v_cache, "v_cache");
    TORCH_CHECK(k_cache.dim() == 3 && v_cache.sizes() == k_cache.sizes(), "caches must be [heads, max_len, head_dim]");
    const int64_t n_heads = k_cache.size(0), max_len = k_cache.size(1), head_dim = k_cache.size(2);
    TORCH_CHECK(q.numel() == n_heads * head_dim && k.numel() == q.numel() && v.numel() == q.numel(), "bad q/k/v size");
    TORCH_CHECK(cos_table.is_cuda() && cos_table.dtype() == at::kFloat && cos_table.is_contiguous() &&
                    cos_table.numel() == max_len * (head_dim / 2) && sin_table.is_cuda() &&
                    sin_table.dtype() == at::kFloat && sin_table.is_contiguous() &&
                    sin_table.numel() == cos_table.numel(),
                "cos/sin tables must be contiguous float32 GPU tensors [max_len, head_dim/2]");
    TORCH_CHECK(position.is_cuda() && position.dtype() == at::kLong && position.numel() == 1, "bad position");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
    at::Tensor out = at::empty_like(q);
    check_rc(macko_decode_rope_attention_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), cos_table.data_ptr<float>(),
                                             sin_table.data_ptr<float>(), position.data_ptr<int64_t>(),
                                             k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), (int32_t)n_heads,
                                             (int32_t)head_dim, (int32_t)max_len, (float)scale,
                                             (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
             "decode_rope_attention");
    return out;
}

}  // namespace

TORCH_LIBRARY(macko_spmv, m)
{
    // same schema string as the upstream package
    m.def("multiply(Tensor M_values, Tensor M_deltas, Tensor M_row_indices, int M_rows, int M_cols, Tensor V) -> Tensor");
    m.def("multiply_batched(Tensor M_values, Tensor M_deltas, Tensor M_row_indices, int M_rows, int M_cols, "
          "Tensor X) -> Tensor");
    m.def("multiply_axpby(Tensor M_values, Tensor M_deltas, Tensor M_row_indices, int M_rows, int M_cols, "
          "Tensor V, Tensor(a!) C, float alpha, float beta) -> ()");
    m.def("plan(Tensor M_row_indices, int M_rows, int M_cols, int padded_entries) -> Tensor");
    m.def("multiply_planned(Tensor M_values, Tensor M_deltas, Tensor M_row_indices, int M_rows, int M_cols, "
          "Tensor V, Tensor plan) -> Tensor");
    m.def("multiply_axpby_planned(Tensor M_values, Tensor M_deltas, Tensor M_row_indices, int M_rows, int M_cols, "
          "Tensor V, Tensor(a!) C, float alpha, float beta, Tensor plan) -> ()");
    m.def("compress(Tensor M) -> (Tensor, Tensor, Tensor, int, int)");
    m.def("compress_int8(Tensor M) -> (Tensor, Tensor, Tensor, int, int)");
    m.def("multiply_int8(Tensor M_values, Tensor M_deltas, Tensor M_row_indices, int M_rows, int M_cols, "
          "Tensor V) -> Tensor");
    m.def("multiply_int8_axpby(Tensor M_values, Tensor M_deltas, Tensor M_row_indices, int M_rows, int M_cols, "
          "Tensor V, Tensor(a!) C, float alpha, float beta) -> ()");
    m.def("decode_rmsnorm(Tensor x, Tensor weight, float eps) -> Tensor");
    m.def("decode_rope_append(Tensor q, Tensor k, Tensor v, Tensor cos_table, Tensor sin_table, Tensor position, "
          "Tensor(a!) k_cache, Tensor(b!) v_cache) -> Tensor");
    m.def("decode_attention(Tensor q, Tensor k_cache, Tensor v_cache, Tensor position, float scale) -> Tensor");
    m.def("decode_silu_mul(Tensor gate, Tensor up) -> Tensor");
    m.def("multiply_rmsnorm(Tensor M_values, Tensor M_deltas, Tensor M_row_indices, int M_rows, int M_cols, "
          "Tensor V, Tensor norm_weight, float eps) -> Tensor");
    m.def("multiply_silu_mul_axpby(Tensor M_values, Tensor M_deltas, Tensor M_row_indices, int M_rows, int M_cols, "
          "Tensor gate, Tensor up, Tensor(a!) C, float alpha, float beta) -> ()");
    m.def("decode_rope_attention(Tensor q, Tensor k, Tensor v, Tensor cos_table, Tensor sin_table, Tensor position, "
          "Tensor(a!) k_cache, Tensor(b!) v_cache, float scale) -> Tensor");
    m.def("decompress(Tensor M_values, Tensor M_deltas, Tensor M_row_indices, int M_rows, int M_cols) -> Tensor");
}

TORCH_LIBRARY_IMPL(macko_spmv, CUDA, m)
{
    m.impl("multiply", &multiply_hip);
    m.impl("multiply_batched", &multiply_batched_hip);
    m.impl("multiply_axpby", &multiply_axpby_hip);
    m.impl("plan", &plan_hip);
    m.impl("multiply_planned", &multiply_planned_hip);
    m.impl("multiply_axpby_planned", &multiply_axpby_planned_hip);
    m.impl("compress", &compress_hip);
    m.impl("compress_int8", &compress_int8_hip);
    m.impl("multiply_int8", &multiply_int8_hip);
    m.impl("multiply_int8_axpby", &multiply_int8_axpby_hip);
    m.impl("decode_rmsnorm", &decode_rmsnorm_hip);
    m.impl("decode_rope_append", &decode_rope_append_hip);
    m.impl("decode_attention", &decode_attention_hip);
    m.impl("decode_silu_mul", &decode_silu_mul_hip);
    m.impl("multiply_rmsnorm", &multiply_rmsnorm_hip);
    m.impl("multiply_silu_mul_axpby", &multiply_silu_mul_axpby_hip);
    m.impl("decode_rope_attention", &decode_rope_attention_hip);
    m.impl("decompress", &decompress_hip);
}

TORCH_LIBRARY_IMPL(macko_spmv, CPU, m)
{
    m.impl("compress", &compress_cpu);
    m.impl("compress_int8", &compress_int8_cpu);
}
