"""MACKO sparse matrix-vector multiplication for AMD MI355X (gfx950).

Drop-in for the Python surface of the upstream `macko_spmv` package
(src/macko_spmv/__init__.py:110-149):

    compressed = compress(M)             # 5-tuple (values, deltas, row_indices, rows, cols)
    y = multiply(compressed, V)          # fp16 [rows]
    compressed = move_to_device(compressed, "cuda")

`multiply` goes through the torch operator `torch.ops.macko_spmv.multiply` (same schema as
upstream, fake-tensor implementation registered, usable under torch.compile).  Both functions
run hand-written HIP kernels through the C ABI in include/macko_hip.h; there is no CPU
implementation, and importing this package fails if the native libraries cannot be loaded.
"""
import ctypes
import os
import types

import torch

from . import _build

__version__ = "0.2.0"
LIB_NAME = "macko_spmv"


def _load_native():
    hip_path, torch_path = _build.lib_paths()
    if not _build.is_current():
        # first use, or the sources have changed since the libraries were built: compile in place,
        # like the upstream package's JIT step at import (src/macko_spmv/__init__.py:14-102)
        _build.build_all()
    try:
        hip = ctypes.CDLL(hip_path, mode=ctypes.RTLD_GLOBAL)
        torch.ops.load_library(torch_path)
    except OSError as exc:  # no silent fallback: the HIP path is the only path
        raise ImportError(
            f"macko_spmv_amd: cannot load its native libraries ({hip_path}, {torch_path}): {exc}. "
            "Rebuild them with `python macko_spmv_amd/_build.py`."
        ) from exc
    return hip, hip_path, torch_path


_hip_lib, HIP_LIBRARY_PATH, TORCH_LIBRARY_PATH = _load_native()


@torch.library.register_fake("macko_spmv::multiply")
def _multiply_fake(M_values, M_deltas, M_row_indices, M_rows, M_cols, V):
    # upstream fake implementation: src/macko_spmv/__init__.py:105-107
    return torch.empty((M_rows,), device=M_values.device, dtype=M_values.dtype)


@torch.library.register_fake("macko_spmv::multiply_planned")
def _multiply_planned_fake(M_values, M_deltas, M_row_indices, M_rows, M_cols, V, plan):
    return torch.empty((M_rows,), device=M_values.device, dtype=M_values.dtype)


@torch.library.register_fake("macko_spmv::multiply_axpby_planned")
def _multiply_axpby_planned_fake(M_values, M_deltas, M_row_indices, M_rows, M_cols, V, C, alpha, beta, plan):
    return None


@torch.library.register_fake("macko_spmv::multiply_batched")
def _multiply_batched_fake(M_values, M_deltas, M_row_indices, M_rows, M_cols, X):
    return torch.empty((X.shape[0], M_rows), device=M_values.device, dtype=M_values.dtype)


@torch.library.register_fake("macko_spmv::multiply_axpby")
def _multiply_axpby_fake(M_values, M_deltas, M_row_indices, M_rows, M_cols, V, C, alpha, beta):
    return None


@torch.library.register_fake("macko_spmv::multiply_rmsnorm")
def _multiply_rmsnorm_fake(M_values, M_deltas, M_row_indices, M_rows, M_cols, V, norm_weight, eps):
    return torch.empty((M_rows,), device=M_values.device, dtype=M_values.dtype)


@torch.library.register_fake("macko_spmv::multiply_silu_mul_axpby")
def _multiply_silu_mul_axpby_fake(M_values, M_deltas, M_row_indices, M_rows, M_cols, gate, up, C, alpha, beta):
    return None


@torch.library.register_fake("macko_spmv::decode_rope_attention")
def _decode_rope_attention_fake(q, k, v, cos_table, sin_table, position, k_cache, v_cache, scale):
    return torch.empty_like(q)


@torch.library.register_fake("macko_spmv::decode_rmsnorm")
def _decode_rmsnorm_fake(x, weight, eps):
    return torch.empty_like(x)


@torch.library.register_fake("macko_spmv::decode_rope_append")
def _decode_rope_append_fake(q, k, v, cos_table, sin_table, position, k_cache, v_cache):
    return torch.empty_like(q)


@torch.library.register_fake("macko_spmv::decode_attention")
def _decode_attention_fake(q, k_cache, v_cache, position, scale):
    return torch.empty_like(q)


@torch.library.register_fake("macko_spmv::decode_silu_mul")
def _decode_silu_mul_fake(gate, up):
    return torch.empty_like(gate)


# compress and compress_int8 have no fake implementation on purpose: the length of their outputs
# depends on the data and the call waits for the GPU in the middle, so they run eagerly only
# (torch.compile breaks the graph around them).


@torch.library.register_fake("macko_spmv::multiply_int8")
def _multiply_int8_fake(M_values, M_deltas, M_row_indices, M_rows, M_cols, V):
    return torch.empty((M_rows,), device=V.device, dtype=V.dtype)


@torch.library.register_fake("macko_spmv::multiply_int8_axpby")
def _multiply_int8_axpby_fake(M_values, M_deltas, M_row_indices, M_rows, M_cols, V, C, alpha, beta):
    return None


@torch.library.register_fake("macko_spmv::decompress")
def _decompress_fake(M_values, M_deltas, M_row_indices, M_rows, M_cols):
    return torch.empty((M_rows, M_cols), device=M_values.device, dtype=M_values.dtype)


def _multiply_vmap(info, in_dims, M_values, M_deltas, M_row_indices, M_rows, M_cols, V):
    """torch.vmap over the vector argument (the way the upstream LLM runner lifts the operator to a
    sequence of tokens, python_scripts/util_run_pruned_llm.py:109-113) becomes one batched product."""
    if any(d is not None for d in in_dims[:5]) or in_dims[5] is None:
        raise NotImplementedError("macko_spmv::multiply: vmap is supported over V only")
    X = V.movedim(in_dims[5], 0).reshape(info.batch_size, -1).contiguous()
    return torch.ops.macko_spmv.multiply_batched.default(M_values, M_deltas, M_row_indices, M_rows, M_cols, X), 0


torch.library.register_vmap("macko_spmv::multiply", _multiply_vmap)


def _multiply_planned_vmap(info, in_dims, M_values, M_deltas, M_row_indices, M_rows, M_cols, V, plan):
    # the batched product has no use for the single-vector launch's cuts
    if in_dims[6] is not None:
        raise NotImplementedError("macko_spmv::multiply_planned: vmap is supported over V only")
    return _multiply_vmap(info, in_dims[:6], M_values, M_deltas, M_row_indices, M_rows, M_cols, V)


torch.library.register_vmap("macko_spmv::multiply_planned", _multiply_planned_vmap)


# A compressed matrix on the GPU carries, as an attribute of its row_indices tensor, where every wave
# of the product's launch starts (a "plan", torch.ops.macko_spmv.plan): `multiply` then has no rows to
# search for.  The tuple keeps the upstream layout; a tuple without the attribute (tensors cloned, moved
# or made elsewhere) multiplies the same, bit for bit, searching row_indices as it goes.  The tensors of
# a compressed matrix are not to be modified in place.
_PLAN_ATTRIBUTE = "_macko_spmv_plan"


def attach_plan(compressed):
    """Prepare the product's cuts for a compressed fp16 matrix on the GPU (once per matrix; `compress`
    and `move_to_device` call this).  Returns `compressed`."""
    values, _, row_indices, rows, cols = compressed[:5]
    if row_indices.is_cuda and values.dtype == torch.float16:
        plan = torch.ops.macko_spmv.plan.default(row_indices, rows, cols, values.numel())
        setattr(row_indices, _PLAN_ATTRIBUTE, plan if plan.numel() else None)
    return compressed


def _plan_of(compressed):
    plan = getattr(compressed[2], _PLAN_ATTRIBUTE, None)
    return plan if plan is not None and plan.device == compressed[2].device else None


def move_to_device(compressed, device):
    """Move the three tensors of a compressed matrix (src/macko_spmv/__init__.py:110-117)."""
    return attach_plan((
        compressed[0].to(device=device),
        compressed[1].to(device=device),
        compressed[2].to(device=device),
        compressed[3],
        compressed[4],
    ))


def compress(M):
    """Dense fp16 matrix -> (values fp16[P], deltas uint8[P/2], row_indices int32[R+1], R, C).

    Same routing as upstream (src/macko_spmv/__init__.py:120-131): a GPU tensor yields GPU
    tensors, a CPU tensor yields CPU tensors, other devices raise NotImplementedError.  In both
    supported cases the arrays are produced by the HIP compressor (a CPU tensor is staged
    through the current GPU).
    """
    assert M.is_contiguous()
    if M.device.type in ("cuda", "cpu"):
        return attach_plan(tuple(torch.ops.macko_spmv.compress.default(M)))
    raise NotImplementedError()


def multiply(compressed_M, V):
    """y = M @ V for a compressed M; fp16 in, fp32 accumulation, fp16 out
    (src/macko_spmv/__init__.py:134-149)."""
    assert compressed_M[0].is_cuda
    assert compressed_M[1].is_cuda
    assert compressed_M[2].is_cuda
    assert V.is_cuda
    assert V.is_contiguous()
    plan = _plan_of(compressed_M)
    if plan is not None:
        return torch.ops.macko_spmv.multiply_planned.default(*compressed_M[:5], V, plan)
    return torch.ops.macko_spmv.multiply.default(
        compressed_M[0],
        compressed_M[1],
        compressed_M[2],
        compressed_M[3],
        compressed_M[4],
        V,
    )


def multiply_batched(compressed_M, X):
    """Y[b] = M @ X[b] for X of shape (batch, cols) -> (batch, rows).  The matrix is read once per
    group of up to eight vectors.  Upstream has only the single-vector operator and maps it over
    the batch dimension (python_scripts/util_run_pruned_llm.py:112-118)."""
    assert compressed_M[0].is_cuda and X.is_cuda
    assert X.dim() == 2 and X.is_contiguous()
    return torch.ops.macko_spmv.multiply_batched.default(*compressed_M[:5], X)


def multiply_axpby(compressed_M, V, C, alpha=1.0, beta=0.0):
    """In place C = alpha * (M @ V) + beta * C: the epilogue of the upstream kernel's
    reuse_value_from_c instantiation (src/macko_spmv/cuda/kernels.cuh:113-118)."""
    assert compressed_M[0].is_cuda and V.is_cuda and C.is_cuda
    assert V.is_contiguous() and C.is_contiguous()
    plan = _plan_of(compressed_M)
    if plan is not None:
        torch.ops.macko_spmv.multiply_axpby_planned.default(*compressed_M[:5], V, C, float(alpha), float(beta), plan)
        return C
    torch.ops.macko_spmv.multiply_axpby.default(
        compressed_M[0], compressed_M[1], compressed_M[2], compressed_M[3], compressed_M[4], V, C,
        float(alpha), float(beta),
    )
    return C


def multiply_rmsnorm(compressed_M, V, norm_weight, eps):
    """M @ rmsnorm(V) with rmsnorm(V) = fp16(V * rsqrt(mean(V^2) + eps) * norm_weight), the norm
    applied while the product stages its input (no launch, no round trip through memory for it).
    Needs cols % 8 == 0 and a vector that fits in LDS.  No upstream counterpart."""
    assert compressed_M[0].is_cuda and V.is_cuda and norm_weight.is_cuda
    return torch.ops.macko_spmv.multiply_rmsnorm.default(*compressed_M[:5], V, norm_weight, float(eps))


def multiply_silu_mul_axpby(compressed_M, gate, up, C, alpha=1.0, beta=0.0):
    """In place C = alpha * M @ (silu(gate) * up) + beta * C: the gated activation of a Llama MLP
    applied while the down projection stages its input.  Same limits as multiply_rmsnorm."""
    assert compressed_M[0].is_cuda and gate.is_cuda and up.is_cuda and C.is_cuda
    torch.ops.macko_spmv.multiply_silu_mul_axpby.default(*compressed_M[:5], gate, up, C, float(alpha), float(beta))
    return C


def compress_int8(M):
    """Dense int8 matrix -> (values int8[P], deltas uint8[P/2], row_indices int32[R+1], R, C).

    The int8 twin of compress (compress_rows_int8_cpu, src/macko_spmv/cuda/cpu_compressor.cuh:75-117;
    upstream has no Python entry for it).  Unlike the fp16 format it keeps the padding entries
    behind a row's last non-zero.  Device routing as in compress.
    """
    assert M.is_contiguous()
    if M.device.type in ("cuda", "cpu"):
        return tuple(torch.ops.macko_spmv.compress_int8.default(M))
    raise NotImplementedError()


def multiply_int8(compressed_M, V):
    """y = M @ V for an int8-compressed M and an fp16 V; fp32 accumulation, fp16 out
    (macko_spmv_int8<false>, src/macko_spmv/cuda/kernels.cuh:126-216)."""
    assert compressed_M[0].is_cuda
    assert compressed_M[1].is_cuda
    assert compressed_M[2].is_cuda
    assert V.is_cuda
    assert V.is_contiguous()
    return torch.ops.macko_spmv.multiply_int8.default(*compressed_M[:5], V)


def multiply_int8_axpby(compressed_M, V, C, alpha=1.0, beta=0.0):
    """In place C = alpha * (M @ V) + beta * C with int8 values (macko_spmv_int8<true>,
    src/macko_spmv/cuda/kernels.cuh:208-211)."""
    assert compressed_M[0].is_cuda and V.is_cuda and C.is_cuda
    assert V.is_contiguous() and C.is_contiguous()
    torch.ops.macko_spmv.multiply_int8_axpby.default(*compressed_M[:5], V, C, float(alpha), float(beta))
    return C


def decompress(compressed_M):
    """Dense fp16 matrix back from a compressed one (GPU tensors).  Not part of the upstream API."""
    assert compressed_M[0].is_cuda
    return torch.ops.macko_spmv.decompress.default(*compressed_M[:5])


# Names some upstream callers reach for (src/macko_spmv/__init__.py:36,90,141).
__compressor_lib = types.SimpleNamespace(cpu_compress=lambda M: tuple(torch.ops.macko_spmv.compress.default(M)))
__multiply_lib = types.SimpleNamespace(macko_spmv_launcher=torch.ops.macko_spmv.multiply.default)
