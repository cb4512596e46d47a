"""torch.compile through the two custom operators on the real library (reference
src/risa_attention/dense.py:14-77 registers the same operators so that compiled graphs
keep one opaque node per attention call)."""

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_compiled_graph_equals_eager(risa, mode):
    torch.manual_seed(7)
    q = torch.randn(1, 4, 300, 128, device="cuda", dtype=torch.bfloat16)
    k = torch.randn(1, 2, 1300, 128, device="cuda", dtype=torch.bfloat16)
    v = torch.randn(1, 2, 1300, 128, device="cuda", dtype=torch.bfloat16)
    key_mask = torch.ones(1, 1, 1, 1300, device="cuda", dtype=torch.bool)
    key_mask[..., 900:] = False
    row_mask = torch.ones(300, 1300, device="cuda", dtype=torch.bool)
    row_mask[0] = False
    row_mask[1:, 3::7] = False

    def plain(q, k, v):
        return risa.int8_attention(q * 1.0, k, v, v_quantization=mode) + 0.0

    def causal(q, k, v):
        return risa.int8_attention(q, k, v, v_quantization=mode, is_causal=True, scale=0.05)

    def masked(q, k, v, mask):
        return risa.int8_attention(q, k, v, attn_mask=mask, v_quantization=mode)

    for function, arguments in ((plain, (q, k, v)), (causal, (q, k, v)), (masked, (q, k, v, key_mask)),
                                (masked, (q, k, v, row_mask))):
        eager = function(*arguments)
        compiled = torch.compile(function, backend="aot_eager", fullgraph=True)
        for _ in range(2):  # the second call replays the cached graph
            assert torch.equal(compiled(*arguments), eager), function.__name__


def test_operator_recorded_by_make_fx_runs_the_kernel(risa):
    """A graph recorded with real tensors holds the operator node, and running the graph
    module launches the kernel again (the ctypes call is not traced away)."""
    from torch.fx.experimental.proxy_tensor import make_fx

    torch.manual_seed(8)
    q = torch.randn(1, 2, 200, 64, device="cuda", dtype=torch.float16)
    k = torch.randn(1, 2, 500, 64, device="cuda", dtype=torch.float16)
    v = torch.randn(1, 2, 500, 64, device="cuda", dtype=torch.float16)
    graph = make_fx(lambda q, k, v: risa.int8_attention(q, k, v), tracing_mode="real")(q, k, v)
    targets = [str(node.target) for node in graph.graph.nodes if node.op == "call_function"]
    assert any("risa_attention.int8_attention" in name for name in targets), targets
    other = torch.randn_like(q)
    assert torch.equal(graph(other, k, v), risa.int8_attention(other, k, v))
