"""The ComfyUI adapter on the real library: ComfyUI-shaped tensors in, the same numbers
out as the direct calls, and a sampling run that builds each pattern once and reuses it."""

import pytest
import torch

from tests.test_comfyui_adapter import Container, node

pytestmark = pytest.mark.gpu


def comfy_tensors(batch, tokens, heads, channels, seed, kv_heads=None):
    generator = torch.Generator(device="cpu").manual_seed(seed)
    make = lambda h: torch.randn(batch, tokens, h * channels, generator=generator).to("cuda", torch.bfloat16)
    return make(heads), make(kv_heads or heads), make(kv_heads or heads)


def head_major(tensor, heads):
    batch, tokens, width = tensor.shape
    return tensor.reshape(batch, tokens, heads, width // heads).transpose(1, 2)


def test_dense_adapter_matches_direct_call(risa):
    attention = node.make_int8_attention_function(risa)
    q, k, v = comfy_tensors(2, 300, 8, 64, 1, kv_heads=2)
    mask = torch.ones(300, 300, dtype=torch.bool, device="cuda").tril()
    for kwargs in ({}, {"mask": mask}, {"scale": 0.2}):
        output = attention(q, k, v, heads=8, enable_gqa=True, **kwargs)
        direct = risa.int8_attention(head_major(q, 8), head_major(k, 2), head_major(v, 2),
                                     scale=kwargs.get("scale"), attn_mask=kwargs.get("mask"))
        assert output.shape == q.shape
        assert torch.equal(head_major(output, 8), direct)
        boxed = attention.container_function(Container(q.clone()), Container(k.clone()), Container(v.clone()),
                                             heads=8, enable_gqa=True, **kwargs)
        assert torch.equal(boxed, output)
    kept = attention(head_major(q, 8), head_major(k, 2), head_major(v, 2), heads=8, skip_reshape=True,
                     skip_output_reshape=True)
    assert kept.shape == (2, 8, 300, 64)


def test_sampling_run_builds_patterns_once_and_reuses_them(risa):
    state = node._SparsePatternState(theta=0.9)
    attention = node.make_sparse_attention_function(risa, state)
    q, k, v = comfy_tensors(1, 2048, 4, 128, 2)
    k = k * 3  # peaked attention: the patterns drop most tiles
    dense = risa.int8_attention(head_major(q, 4), head_major(k, 4), head_major(v, 4))

    def sampling_run():
        outputs = []
        for step in range(3):
            for branch in ("positive", "negative"):
                outputs.append(state.diffusion_model_wrapper(
                    lambda **_: [attention(q, k, v, heads=4), attention(q, k, v, heads=4)],
                    transformer_options={"uuids": [branch]}))
            if step == 0:
                assert len(state.patterns) == 4  # 2 branches x 2 attention calls
        return outputs

    outputs = state.outer_sample_wrapper(sampling_run)
    assert state.patterns == {}
    def distance(output):
        return ((head_major(output, 4).float() - dense.float()).norm() / dense.float().norm()).item()

    # Construction returns the dense result (from the capturing kernel, whose FP32
    # summation order differs from the small-launch kernel in the last bit).
    assert distance(outputs[0][0]) < 1e-3
    for later in outputs[2:]:
        for output in later:
            assert 1e-3 < distance(output) < 0.35  # theta = 0.9 drops up to 10 % of the mass per block
    # Outside a sampling run the same callable is plain dense attention.
    assert torch.equal(head_major(attention(q, k, v, heads=4), 4), dense)

    state.begin_session()
    state.begin_forward({})
    boxed = attention.container_function(Container(q.clone()), Container(k.clone()), Container(v.clone()), heads=4)
    pattern = next(iter(state.patterns.values()))
    assert 0.05 <= pattern.sparsity < 1 and pattern.retained_mass_target == 0.9
    state.end_forward()
    state.begin_forward({})
    reused = attention.container_function(Container(q.clone()), Container(k.clone()), Container(v.clone()), heads=4)
    state.end_forward()
    state.end_session()
    assert distance(boxed) < 1e-3
    assert torch.equal(reused, outputs[2][0])
