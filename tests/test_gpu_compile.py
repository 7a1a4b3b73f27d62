"""torch.compile through the registered fakes.  The reference registers a fake (meta) kernel for
``moe::m_grouped_gemm`` so that the op can sit inside a compiled graph (gemm/BF16/m_grouped_gemm_TMA.py:450-462); the
FP8 per-channel op is a ``triton_op`` there for the same purpose (gemm/FP8/m_grouped_gemm_channel_expert.py:139).
Here both are custom ops over the HIP library: a compiled function that calls them must trace in one graph
(``fullgraph=True``: no graph break at the op), take its output shapes and dtypes from the fakes, and return what
the eager call returns, bit for bit.  The ``aot_eager`` backend runs Dynamo's tracing, fake-tensor propagation and
AOT autograd's functionalisation -- everything that consults the fake -- and leaves code generation for the
surrounding pointwise work out, so the test needs no code generator on the box."""
import pytest
import torch

from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_TMA import m_grouped_gemm
from triton_grouped_gemm_amd.gemm.FP8.m_grouped_gemm_channel_expert import gmm_fp8_act_per_channel_w_per_expert

pytestmark = pytest.mark.gpu


def test_m_grouped_gemm_compiles_in_one_graph(dev):
    torch.manual_seed(7)
    sizes = torch.tensor([64, 0, 130, 62], dtype=torch.int32, device=dev)
    a = (torch.randn(256, 128, device=dev) / 11).to(torch.bfloat16)
    b = (torch.randn(4, 264, 128, device=dev) / 11).to(torch.bfloat16)

    def layer(x, w, s):
        y = m_grouped_gemm(x * 2, w, s, True)        # pointwise work either side of the op, as a caller would have
        return torch.nn.functional.silu(y.float()).to(torch.bfloat16)

    torch._dynamo.reset()
    compiled = torch.compile(layer, fullgraph=True, backend="aot_eager")
    got = compiled(a, b, sizes)
    want = layer(a, b, sizes)
    assert got.shape == (256, 264) and got.dtype == torch.bfloat16
    assert torch.equal(got, want)
    # other group sizes (read on the device) and the other weight layout through the same compiled function family
    sizes2 = torch.tensor([1, 255, 0, 0], dtype=torch.int32, device=dev)
    assert torch.equal(compiled(a, b, sizes2), layer(a, b, sizes2))
    bt = b.transpose(1, 2).contiguous()
    nn_layer = torch.compile(lambda x, w, s: m_grouped_gemm(x, w, s, False), fullgraph=True, backend="aot_eager")
    assert torch.equal(nn_layer(a, bt, sizes), m_grouped_gemm(a, bt, sizes, False))


def test_fp8_per_channel_op_compiles_in_one_graph(dev):
    torch.manual_seed(8)
    sizes = torch.tensor([128, 16, 0, 112], dtype=torch.int32, device=dev)
    a = torch.randn(256, 256, device=dev).to(torch.float8_e4m3fn)
    w = torch.randn(4, 136, 256, device=dev).to(torch.float8_e4m3fn)
    sa = torch.rand(256, 1, device=dev) + 0.5
    sb = torch.rand(4 * 136, device=dev) + 0.5

    def layer(x, xs, ww, ws, s):
        return gmm_fp8_act_per_channel_w_per_expert(x, xs * 1.0, ww, ws, s, torch.bfloat16) + 1

    torch._dynamo.reset()
    compiled = torch.compile(layer, fullgraph=True, backend="aot_eager")
    got = compiled(a, sa, w, sb, sizes)
    assert got.shape == (256, 136) and got.dtype == torch.bfloat16
    assert torch.equal(got, layer(a, sa, w, sb, sizes))
    # the default output dtype comes from the fake as well
    half = torch.compile(lambda x, xs, ww, ws, s: gmm_fp8_act_per_channel_w_per_expert(x, xs, ww, ws, s),
                         fullgraph=True, backend="aot_eager")
    assert half(a, sa, w, sb, sizes).dtype == torch.float16
