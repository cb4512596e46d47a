"""NRMSE against FP32 SDPA over the reference's dense table (reference README.md:115-123):
B=1, Hq=16, Hkv=4, D=128, bf16 N(0,1) inputs, N = 512 ... 32K, both V modes, mean over seeds
0/1/2 of the record of benchmarks/common.py:148-164.  The bar is the README's figure to its
printed precision (figure + 0.00005).

The eight cells from N = 4K on meet it.  Up to 2K the three-seed mean sits within +-1.2 % of the
figure with this platform's device generator (512 both modes +1.2 / +1.4 %, 1K absmax +0.6 %, 2K
midpoint_affine +0.4 % of the figure, i.e. 0.1-0.9 % over the bar; 1K midpoint_affine and 2K
absmax under it), with a seed-to-seed spread of up to 1.7 % at 2K.  The test says why instead of
widening the bar for all cells:

* the kernels are not the cause: on the same tensors the oracle's NRMSE equals theirs to five
  digits (asserted below);
* the draws are: the figure moves by several per cent with the tails of the input sample (the
  V and Q/K scales are extreme-value statistics of at most a few thousand draws at these
  lengths).  The same kernels on the CPU generator's bf16 draws of the same seeds meet the
  README's figure in every one of these cells (asserted below); the README's numbers come from a third
  generator (CUDA's) that nothing here can reproduce, and at N >= 8K this build is 0.4-1.6 %
  *below* the README with the device generator.

The allowance for the cells up to 2K is 1.5 % of the figure (ALLOWED); each of them is also
held to the two assertions above.
"""

import numpy as np
import pytest
import torch

from oracle import pipeline as oracle_pipeline

pytestmark = pytest.mark.gpu

# N: (absmax, midpoint_affine), reference README.md:115-123
README_NRMSE = {512: (0.0145, 0.0136), 1024: (0.0149, 0.0140), 2048: (0.0158, 0.0148), 4096: (0.0161, 0.0151),
                8192: (0.0166, 0.0155), 16384: (0.0168, 0.0156), 32768: (0.0169, 0.0157)}
PRINTED_PRECISION = 0.00005
MODES = ("absmax", "midpoint_affine")
ALLOWED = {(length, mode): 0.015 for length in (512, 1024, 2048) for mode in MODES}
SEEDS = (0, 1, 2)


def device_inputs(length, seed):
    """Tensors drawn on the device in the order q, k, v (reference benchmarks/common.py:105-131)."""
    generator = torch.Generator(device="cuda").manual_seed(seed)
    draw = lambda heads: torch.randn((1, heads, length, 128), generator=generator, device="cuda", dtype=torch.bfloat16)
    return draw(16), draw(4), draw(4)


def host_inputs(length, seed):
    generator = torch.Generator().manual_seed(seed)
    draw = lambda heads: torch.randn((1, heads, length, 128), generator=generator, dtype=torch.bfloat16).cuda()
    return draw(16), draw(4), draw(4)


def fp32_reference(q, k, v, chunk=2048):
    keys = k.float().repeat_interleave(4, 1).transpose(-1, -2)
    values = v.float().repeat_interleave(4, 1)
    out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    for start in range(0, q.shape[2], chunk):
        scores = q[:, :, start:start + chunk].float() @ keys * 128 ** -0.5
        out[:, :, start:start + chunk] = torch.softmax(scores, dim=-1) @ values
    return out


def nrmse(actual, reference):
    error = actual.float() - reference
    return (error.pow(2).mean().sqrt() / reference.pow(2).mean().sqrt().clamp_min(1e-12)).item()


@pytest.mark.parametrize("length", sorted(README_NRMSE))
def test_nrmse_against_fp32_sdpa_meets_the_readme_table(risa, length):
    measured = {mode: [] for mode in MODES}
    from_oracle = {mode: [] for mode in MODES}
    for seed in SEEDS:
        q, k, v = device_inputs(length, seed)
        reference = fp32_reference(q, k, v)
        for mode in MODES:
            measured[mode].append(nrmse(risa.int8_attention(q, k, v, v_quantization=mode), reference))
            if (length, mode) in ALLOWED:
                expected = oracle_pipeline.int8_attention(q.float().cpu().numpy(), k.float().cpu().numpy(),
                                                          v.float().cpu().numpy(), v_quantization=mode)
                from_oracle[mode].append(nrmse(torch.from_numpy(expected).cuda(), reference))
        del reference
    for mode, figure in zip(MODES, README_NRMSE[length]):
        mean = float(np.mean(measured[mode]))
        print(f"N={length} {mode}: NRMSE {mean:.5f} (seeds {[round(x, 5) for x in measured[mode]]}), README {figure}", flush=True)
        bar = figure + PRINTED_PRECISION
        if (length, mode) not in ALLOWED:
            assert mean < bar, (length, mode, mean)
            continue
        assert mean < figure * (1.0 + ALLOWED[(length, mode)]), (length, mode, mean)
        # the same tensors through the oracle: the figure is the algorithm's, not the kernels'
        np.testing.assert_allclose(measured[mode], from_oracle[mode], rtol=0, atol=2e-5)
        # the same seeds from the host generator: the README's figure is met
        host = []
        for seed in SEEDS:
            q, k, v = host_inputs(length, seed)
            host.append(nrmse(risa.int8_attention(q, k, v, v_quantization=mode), fp32_reference(q, k, v)))
        print(f"N={length} {mode}: host-generator draws {float(np.mean(host)):.5f}", flush=True)
        assert float(np.mean(host)) < bar, (length, mode, host)
