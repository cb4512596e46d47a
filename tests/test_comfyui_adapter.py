"""Host contracts of the ComfyUI adapter (no GPU, no ComfyUI): node interface, tensor
reshaping incl. grouped-query K/V, pattern lifetime per sampling run / conditioning
branch / call ordinal, scoped wrappers.  Cases after reference
tests/contracts/test_comfyui_node.py:65-172, against a recording stand-in backend."""

import importlib.util
import sys
import threading
from pathlib import Path
from types import SimpleNamespace

import pytest
import torch

PACKAGE_DIR = Path(__file__).resolve().parents[1] / "comfyui-risaattention-amd"


def load_adapter():
    name = "risaattention_amd_comfyui_node"
    if name not in sys.modules:
        spec = importlib.util.spec_from_file_location(name, PACKAGE_DIR / "__init__.py",
                                                      submodule_search_locations=[str(PACKAGE_DIR)])
        package = importlib.util.module_from_spec(spec)
        sys.modules[name] = package
        spec.loader.exec_module(package)
    return sys.modules[name], importlib.import_module(name + ".node")


package, node = load_adapter()


class RecordingBackend:
    """Returns q unchanged and counts which entry point served each call."""

    def __init__(self, sparsity=0.5):
        self.sparsity = sparsity
        self.calls = []
        self.seen = None

    def count(self, name):
        return sum(1 for call in self.calls if call == name)

    @staticmethod
    def int8_attention_is_available():
        return True

    def int8_attention(self, q, k, v, *, scale, attn_mask):
        self.calls.append("dense")
        self.seen = (q.shape, k.shape, v.shape, scale, attn_mask)
        return q

    def sparse_int8_attention(self, q, k, v, pattern, *, scale, output_layout):
        self.calls.append("reuse")
        return q

    def construct_sparse_int8_attention(self, q, k, v, *, theta, scale, output_layout):
        self.calls.append("construct")
        return q, SimpleNamespace(sparsity=self.sparsity, theta=theta)

    def prequantize_int8_attention(self, q, k, v, *, scale, attn_mask):
        self.calls.append("prequantize")
        self.seen = (q.shape, k.shape, v.shape, scale, attn_mask)
        return q

    def int8_attention_from_prequantized(self, packed, *, sparse_pattern=None, output_layout):
        self.calls.append("dense" if sparse_pattern is None else "reuse")
        self.layout = output_layout
        return packed

    def construct_sparse_int8_attention_from_prequantized(self, packed, *, theta, output_layout):
        self.calls.append("construct")
        return packed, SimpleNamespace(sparsity=self.sparsity, theta=theta)


class Container:
    def __init__(self, tensor):
        self.tensor = tensor

    def take(self):
        tensor, self.tensor = self.tensor, None
        return tensor


def fake_model():
    patched = SimpleNamespace(wrappers=[])
    patched.set_model_optimized_attention = lambda function: setattr(patched, "attention", function)
    patched.add_wrapper_with_key = lambda scope, key, function: patched.wrappers.append((scope, key, function))
    return SimpleNamespace(clone=lambda: patched), patched


def test_package_and_node_interface():
    assert package.NODE_CLASS_MAPPINGS == {"RISAAttention": node.RISAAttentionNode}
    assert package.NODE_DISPLAY_NAME_MAPPINGS == {"RISAAttention": "RISA Attention"}
    required = node.RISAAttentionNode.INPUT_TYPES()["required"]
    assert list(required) == ["model", "attention", "theta"]
    assert required["attention"][0] == ["pytorch_attention", "int8_attention", "sparse_int8_attention"]
    assert required["attention"][1]["default"] == "sparse_int8_attention"
    assert required["theta"][1]["default"] == 0.99
    assert (required["theta"][1]["min"], required["theta"][1]["max"]) == (0.9, 1.0)
    assert node.RISAAttentionNode.RETURN_TYPES == ("MODEL",)
    assert node.RISAAttentionNode.FUNCTION == "patch_model"


def test_dense_call_splits_heads_and_keeps_grouped_kv():
    backend = RecordingBackend()
    attention = node.make_int8_attention_function(backend)
    q, k, v = torch.randn(1, 4, 32), torch.randn(1, 6, 16), torch.randn(1, 6, 16)
    output = attention(q, k, v, heads=4, enable_gqa=True, scale=0.25)
    assert backend.seen[:4] == (torch.Size([1, 4, 4, 8]), torch.Size([1, 2, 6, 8]), torch.Size([1, 2, 6, 8]), 0.25)
    assert output.shape == q.shape
    assert torch.equal(output, q)  # split and merge are inverse views


def test_masks_are_lifted_to_four_dimensions():
    backend = RecordingBackend()
    attention = node.make_int8_attention_function(backend)
    q = torch.randn(2, 5, 16)
    attention(q, q, q, heads=2, mask=torch.ones(5, 5, dtype=torch.bool))
    assert backend.seen[4].shape == (1, 1, 5, 5)
    attention(q, q, q, heads=2, mask=torch.zeros(2, 5, 5))
    assert backend.seen[4].shape == (2, 1, 5, 5)


def test_container_calls_quantise_before_releasing_inputs():
    backend = RecordingBackend()
    attention = node.make_int8_attention_function(backend)
    q = torch.randn(1, 3, 2, 8)
    boxes = [Container(q), Container(q.clone()), Container(q.clone())]
    output = attention.container_function(*boxes, heads=3, skip_reshape=True)
    assert all(box.tensor is None for box in boxes)
    assert backend.calls == ["prequantize", "dense"]
    assert backend.layout == "nhd" and output.shape == (1, 2, 24)
    attention.container_function(Container(q), Container(q), Container(q), heads=3, skip_reshape=True,
                                 skip_output_reshape=True)
    assert backend.layout == "hnd"


def test_pattern_is_built_once_per_call_ordinal_and_then_reused():
    backend = RecordingBackend()
    state = node._SparsePatternState(theta=0.99)
    attention = node.make_sparse_attention_function(backend, state)
    assert attention.sparse_state is state
    q = torch.randn(1, 4, 2048, 8)
    state.begin_session()
    for _ in range(2):
        state.begin_forward({"uuids": ["positive"]})
        attention(q, q, q, heads=4, skip_reshape=True)
        attention(q, q, q, heads=4, skip_reshape=True)
        state.end_forward()
    assert backend.count("construct") == 2 and backend.count("reuse") == 2
    assert len(state.patterns) == 2
    state.end_session()
    assert state.patterns == {}


def test_conditioning_branches_do_not_share_patterns():
    backend = RecordingBackend()
    state = node._SparsePatternState(theta=0.97)
    attention = node.make_sparse_attention_function(backend, state)
    q = torch.randn(1, 4, 2048, 8)
    state.begin_session()
    for branch in ("positive", "negative", "positive"):
        state.begin_forward({"uuids": [branch]})
        attention(q, q, q, heads=4, skip_reshape=True)
        state.end_forward()
    assert [pattern.theta for pattern in state.patterns.values()] == [0.97, 0.97]
    state.end_session()
    assert backend.count("construct") == 2 and backend.count("reuse") == 1


def test_ineligible_calls_run_dense_and_keep_the_ordinal_moving():
    backend = RecordingBackend()
    state = node._SparsePatternState(theta=0.99)
    attention = node.make_sparse_attention_function(backend, state)
    q, cross = torch.randn(1, 2, 256, 8), torch.randn(1, 2, 77, 8)
    attention(q, q, q, heads=2, skip_reshape=True)  # no sampling run open
    assert backend.calls == ["dense"]
    state.begin_session()
    attention(q, q, q, heads=2, skip_reshape=True)  # no forward frame
    state.begin_forward({})
    attention(q, cross, cross, heads=2, skip_reshape=True)                       # ordinal 0: cross-attention
    attention(q, q, q, heads=2, skip_reshape=True, mask=torch.ones(256, 256))    # ordinal 1: masked
    attention(q, q, q, heads=2, skip_reshape=True)                               # ordinal 2: eligible
    state.end_forward()
    assert backend.calls == ["dense", "dense", "dense", "dense", "construct"]
    assert [key[1] for key in state.patterns] == [2]
    state.end_session()


def test_nearly_dense_patterns_are_served_dense_for_the_rest_of_the_run():
    backend = RecordingBackend(sparsity=0.01)
    state = node._SparsePatternState(theta=0.999)
    attention = node.make_sparse_attention_function(backend, state)
    q = torch.randn(1, 2, 512, 8)
    state.begin_session()
    for _ in range(3):
        state.begin_forward({"cond_or_uncond": [0]})
        attention(q, q, q, heads=2, skip_reshape=True)
        state.end_forward()
    assert backend.calls == ["construct", "dense", "dense"]
    boxes = [Container(q), Container(q), Container(q)]
    state.begin_forward({"cond_or_uncond": [0]})
    attention.container_function(*boxes, heads=2, skip_reshape=True)
    state.end_forward()
    assert backend.calls[-2:] == ["prequantize", "dense"]
    state.end_session()


def test_nested_runs_share_the_store_and_exceptions_close_it():
    state = node._SparsePatternState(theta=0.99)

    def inner():
        state.patterns["kept"] = 1
        return state.outer_sample_wrapper(lambda: dict(state.patterns))

    assert state.outer_sample_wrapper(inner) == {"kept": 1}
    assert state.patterns == {}

    def failing():
        state.patterns["lost"] = 1
        raise KeyError("sampler failed")

    with pytest.raises(KeyError):
        state.outer_sample_wrapper(failing)
    assert state.patterns == {} and state._open_sessions == 0
    seen = state.diffusion_model_wrapper(lambda *a, **k: len(state._frames()), 1,
                                         transformer_options={"uuids": [7]})
    assert seen == 1 and state._frames() == []


def test_forward_frames_are_per_thread():
    state = node._SparsePatternState(theta=0.99)
    state.begin_session()
    state.begin_forward({"uuids": ["main"]})
    q = torch.randn(1, 1, 128, 8)
    result = {}
    worker = threading.Thread(target=lambda: result.update(key=state.next_pattern_key(q, q, q, None, None)))
    worker.start()
    worker.join()
    assert result["key"] is None  # the other thread never entered a forward
    assert state.next_pattern_key(q, q, q, None, 0.5)[:2] == (((("main",)), ()), 0)
    state.end_forward()
    state.end_session()


def test_node_installs_dense_attention_without_sampling_wrappers(monkeypatch):
    model, patched = fake_model()
    monkeypatch.setattr(node, "_load_risa_attention", lambda: RecordingBackend())
    assert node.RISAAttentionNode().patch_model(model, "int8_attention", 0.99) == (patched,)
    assert callable(patched.attention) and callable(patched.attention.container_function)
    assert patched.wrappers == []
    with pytest.raises(ValueError, match="Unsupported attention mode"):
        node.RISAAttentionNode().patch_model(model, "flash", 0.99)


def test_node_installs_sparse_attention_with_both_scopes(monkeypatch):
    model, patched = fake_model()
    scopes = SimpleNamespace(OUTER_SAMPLE="outer", DIFFUSION_MODEL="diffusion")
    real_import = importlib.import_module

    def import_module(name):
        if name == "comfy.patcher_extension":
            return SimpleNamespace(WrappersMP=scopes)
        return real_import(name)

    monkeypatch.setattr(node, "_load_risa_attention", lambda: RecordingBackend())
    monkeypatch.setattr(node.importlib, "import_module", import_module)
    assert node.RISAAttentionNode().patch_model(model, "sparse_int8_attention", 0.95) == (patched,)
    assert [(scope, key) for scope, key, _ in patched.wrappers] == [
        ("outer", "risa_sparse_attention"), ("diffusion", "risa_sparse_attention")]
    assert patched.attention.sparse_state.theta == 0.95


def test_backend_loader_reports_a_missing_gpu(monkeypatch):
    monkeypatch.setattr(node, "_backend_module", None)
    real_import = importlib.import_module

    def import_module(name):
        if name == "risaattention_amd":
            return SimpleNamespace(int8_attention_is_available=lambda: False)
        return real_import(name)

    monkeypatch.setattr(node.importlib, "import_module", import_module)
    with pytest.raises(RuntimeError, match="gfx950"):
        node._load_risa_attention()
