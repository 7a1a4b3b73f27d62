"""Differentiable grouped GEMM: forward, activation gradient and weight gradient on the three native kernels.

Mirrors the autograd wrapper of the reference's baseline extension (grouped_gemm/grouped_gemm/ops.py:12-42):
``gmm(a, b, batch_sizes, trans_b=False, num_sm=-1)`` with

    forward   out = a[rows of g] @ b[g]      (or @ b[g].T with trans_b)        M-grouped, layout NN / NT
    d a       grad @ b[g].T                  (or grad @ b[g])                  M-grouped with trans_b flipped
    d b       a_g.T @ grad_g   ([K, N])      (or grad_g.T @ a_g, [N, K])       K-grouped over the group's rows

``batch_sizes`` may live on the host (as the reference's extension requires) or on the device; a device tensor
is used as is, with no host synchronisation.
"""
import torch

from ._native import require_gpu
from .gemm.BF16.k_grouped_gemm import k_grouped_gemm
from .gemm.BF16.m_grouped_gemm import m_grouped_gemm


def _device_sizes(batch_sizes: torch.Tensor, device: torch.device) -> torch.Tensor:
    if batch_sizes.dtype not in (torch.int32, torch.int64):
        batch_sizes = batch_sizes.to(torch.int64)
    return batch_sizes.to(device, non_blocking=True)


class GroupedGemm(torch.autograd.Function):
    """grouped_gemm/grouped_gemm/ops.py:12-38."""

    @staticmethod
    def forward(ctx, a, b, batch_sizes, trans_b, num_sm=-1):
        if not batch_sizes.is_cuda:
            # the reference asserts this on its host-side sizes; device-resident sizes are not read back
            assert torch.count_nonzero(batch_sizes) != 0, "Input batch_sizes should not be all zeros!"
        require_gpu(a, b)
        sizes = _device_sizes(batch_sizes, a.device)
        ctx.save_for_backward(a, b, sizes)
        ctx.trans_b = bool(trans_b)
        ctx.num_sm = int(num_sm)
        return m_grouped_gemm(a.contiguous(), b.contiguous(), sizes, ctx.trans_b, ctx.num_sm)

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous()
        a, b, sizes = ctx.saved_tensors
        trans_b = ctx.trans_b
        agrad = None
        if ctx.needs_input_grad[0]:
            agrad = m_grouped_gemm(grad, b.contiguous(), sizes, not trans_b, ctx.num_sm)
        bgrad = None
        if ctx.needs_input_grad[1]:
            lhs, rhs = (grad, a) if trans_b else (a, grad)
            bgrad = k_grouped_gemm(lhs.contiguous(), rhs.contiguous(), sizes, numSM=ctx.num_sm)
        return agrad, bgrad, None, None, None


def gmm(a, b, batch_sizes, trans_b=False, num_sm=-1):
    """grouped_gemm/grouped_gemm/ops.py:41-42."""
    return GroupedGemm.apply(a, b, batch_sizes, trans_b, num_sm)


# ---------------------------------------------------------------------------------------------------------------
# MoE token permute / unpermute (grouped_gemm/grouped_gemm/ops.py:52-257)
# ---------------------------------------------------------------------------------------------------------------
import warnings  # noqa: E402

from . import _native  # noqa: E402

_ACT_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float8_e4m3fn: 2, torch.float8_e5m2: 3, torch.float32: 4}
MAX_EXPERTS = 1024


def _act_code(t: torch.Tensor) -> int:
    if t.dtype not in _ACT_CODE:
        raise RuntimeError("Wrong activation tensor type.")  # grouped_gemm/csrc/permute.cu:686
    return _ACT_CODE[t.dtype]


def permute_map(indices: torch.Tensor, num_out_tokens: int = 0, num_experts: int = MAX_EXPERTS,
                counts_dtype: torch.dtype = torch.int32):
    """Stable expert-major order of a ``[num_tokens, topK]`` int32 expert assignment.

    Returns ``(row_id_map [topK * num_tokens] int32, tokens_per_expert [num_experts])``: ``row_id_map[k * T + t]``
    is the permuted row of assignment ``(t, k)`` (-1 when dropped: expert id -1, or row >= ``num_out_tokens`` > 0),
    exactly the map the reference builds from a radix sort (grouped_gemm/csrc/permute.cu:40-101, :541-548);
    ``tokens_per_expert`` is what the grouped GEMMs take as ``size_per_group`` (counts before capacity dropping).
    """
    require_gpu(indices)
    if indices.dim() == 1:
        indices = indices.view(-1, 1)
    tokens, topk = indices.shape
    if not 1 <= num_experts <= MAX_EXPERTS:
        raise ValueError(f"num_experts must be in [1, {MAX_EXPERTS}], got {num_experts}")
    idx = indices.to(torch.int32).contiguous()
    row_id_map = torch.empty(tokens * topk, dtype=torch.int32, device=idx.device)
    counts = torch.empty(num_experts, dtype=counts_dtype, device=idx.device)
    import ctypes
    need = ctypes.c_int64(0)
    _native.call("tgg_moe_sort_workspace_bytes", tokens, topk, num_experts, ctypes.byref(need))
    ws = torch.empty(need.value, dtype=torch.uint8, device=idx.device)
    _native.call("tgg_moe_permute_map", idx.data_ptr(), tokens, topk, num_experts, int(num_out_tokens),
                 row_id_map.data_ptr(), counts.data_ptr(), int(counts_dtype == torch.int64), ws.data_ptr(), need.value,
                 _native.stream_of(idx))
    return row_id_map, counts


def _unpermute_raw(inp, row_id_map, probs, num_tokens, topk):
    out = torch.empty((num_tokens, inp.size(1)), dtype=inp.dtype, device=inp.device)
    _native.call("tgg_moe_unpermute", inp.data_ptr(), out.data_ptr(), row_id_map.data_ptr(),
                 probs.data_ptr() if probs is not None else 0, num_tokens, topk, inp.size(1), _act_code(inp),
                 _native.stream_of(inp))
    return out


def _operand(op: str, name: str, t, device, dtype=None, recommended: str = ""):
    """One tensor argument of a permute / unpermute call brought into the form the kernels take: on the activations'
    device, of the index / probability type, contiguous.  Each adjustment is announced with the warning the
    reference's wrappers give for it (grouped_gemm/grouped_gemm/ops.py:60-92, :178-214), so callers see the same
    diagnostics; nothing is done to a tensor that already conforms."""
    if t.is_cpu:
        warnings.warn(f"The input `{name}` of {op} op is on the device: CPU!")
        t = t.to(device)
    if dtype is not None and t.dtype != dtype:
        warnings.warn(f"The data type of the input `{name}` of {op} op is {t.dtype}! The recommended type is {recommended}.")
        t = t.to(dtype)
    if not t.is_contiguous():
        warnings.warn(f"The input `{name}` of {op} op is discontiguous!")
        t = t.contiguous()
    return t


def _activations(op: str, t):
    if t.is_cpu:
        raise RuntimeError(f"[Error] The input `input_act` of {op} op is on the device: CPU!")
    return _operand(op, "input_act", t, t.device)


class PermuteMoE_topK(torch.autograd.Function):
    """grouped_gemm/grouped_gemm/ops.py:52-160.  The workspace the reference keeps between calls is not needed."""

    @staticmethod
    def forward(ctx, input_act, indices, num_out_tokens, max_token_num, num_experts=MAX_EXPERTS):
        if not input_act.numel():
            return input_act, None
        op = "permute_topK"
        input_act = _activations(op, input_act)
        indices = indices.view(-1, 1) if indices.dim() == 1 else indices
        if input_act.size(0) != indices.size(0):
            raise RuntimeError(f"[Error] {op} op input `indices` shape mismatch! "
                               f"Expect {input_act.size(0)}, but got {indices.size(0)}.")
        indices = _operand(op, "indices", indices, input_act.device, torch.int32, "torch.int32")
        tokens, topk = indices.shape
        row_id_map, _ = permute_map(indices, num_out_tokens, num_experts)
        n_out = num_out_tokens if num_out_tokens > 0 else tokens * topk
        permuted = torch.empty((n_out, input_act.size(1)), dtype=input_act.dtype, device=input_act.device)
        _native.call("tgg_moe_permute_rows", input_act.data_ptr(), permuted.data_ptr(), row_id_map.data_ptr(), tokens,
                     topk, input_act.size(1), _act_code(input_act), _native.stream_of(input_act))
        ctx.row_id_map = row_id_map
        ctx.num_tokens = tokens
        ctx.num_topK = topk
        return permuted, row_id_map

    @staticmethod
    def backward(ctx, permuted_act_grad, _):
        if not permuted_act_grad.numel():
            return permuted_act_grad, None, None, None, None
        grad = permuted_act_grad.contiguous()
        return _unpermute_raw(grad, ctx.row_id_map, None, ctx.num_tokens, ctx.num_topK), None, None, None, None


class UnpermuteMoE_topK(torch.autograd.Function):
    """grouped_gemm/grouped_gemm/ops.py:168-249.  Arithmetic is fp32 with one rounding to the activation type (the
    reference multiplies and accumulates in the activation type)."""

    @staticmethod
    def forward(ctx, input_act, row_id_map, probs=None):
        if not input_act.numel():
            ctx.probs = probs
            return input_act
        op = "unpermute_topK"
        input_act = _activations(op, input_act)
        if probs is not None and row_id_map.size(0) != probs.numel():
            raise RuntimeError(f"[Error] {op} op input `probs` shape mismatch! "
                               f"Expect {row_id_map.size(0)}, but got {probs.size(0) * probs.size(1)}.")
        row_id_map = _operand(op, "row_id_map", row_id_map, input_act.device, torch.int32, "torch.int32")
        if probs is not None:
            probs = _operand(op, "probs", probs, input_act.device, torch.float32, "torch.float32")
        num_tokens, topk = (probs.size(0), probs.size(1)) if probs is not None else (input_act.size(0), 1)
        out = _unpermute_raw(input_act, row_id_map, probs, num_tokens, topk)
        ctx.save_for_backward(input_act, row_id_map, probs)
        ctx.topk = topk
        return out

    @staticmethod
    def backward(ctx, unpermuted_act_grad):
        if not unpermuted_act_grad.numel():
            return unpermuted_act_grad, None, ctx.probs
        grad = unpermuted_act_grad.contiguous()
        input_act, row_id_map, probs = ctx.saved_tensors
        act_grad = prob_grad = None
        if ctx.needs_input_grad[0] or (probs is not None and ctx.needs_input_grad[2]):
            tokens = grad.size(0)
            # rows no kept assignment maps to (possible only after drops) stay unwritten, as in the reference
            act_grad = torch.empty_like(input_act)
            want_pg = probs is not None and ctx.needs_input_grad[2]
            if want_pg:
                prob_grad = torch.empty_like(probs)
            _native.call("tgg_moe_unpermute_bwd", grad.data_ptr(), input_act.data_ptr(), row_id_map.data_ptr(),
                         probs.data_ptr() if probs is not None else 0, act_grad.data_ptr(),
                         prob_grad.data_ptr() if want_pg else 0, tokens, ctx.topk, grad.size(1), _act_code(grad),
                         _native.stream_of(grad))
            if not ctx.needs_input_grad[0]:
                act_grad = None
        return act_grad, None, prob_grad


def permute(input_act, indices, num_out_tokens=None, max_token_num=0, num_experts=MAX_EXPERTS):
    """grouped_gemm/grouped_gemm/ops.py:251-253; ``num_experts`` (optional, <= 1024) sizes the sort's table."""
    num_out_tokens = 0 if num_out_tokens is None else num_out_tokens
    return PermuteMoE_topK.apply(input_act, indices, num_out_tokens, max_token_num, num_experts)


def unpermute(input_act, row_id_map, probs=None):
    """grouped_gemm/grouped_gemm/ops.py:255-256."""
    return UnpermuteMoE_topK.apply(input_act, row_id_map, probs)
