"""CPU tests of the host side: C-ABI exports, input contracts, tile policy, dataclasses,
operator registration (in the spirit of reference tests/contracts/test_risa_attention.py:29-67)."""

import ctypes
import re
from pathlib import Path
from unittest.mock import patch

import pytest
import torch

import risaattention_amd as risa
from risaattention_amd import attend, dense, fp32_patterns, layout, native, policy, types

ROOT = Path(__file__).resolve().parents[1]


def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "risa_hip.h").read_text()
    declared = set(re.findall(r"^(?:int|size_t|void|const char\*)\s+(risa_[a-z0-9_]+)\(", header, re.M))
    assert declared == set(native.SIGNATURES), declared ^ set(native.SIGNATURES)
    library = ctypes.CDLL(str(native.library_path()))
    for name in declared:
        assert hasattr(library, name), name
    assert native.library().risa_abi_version() == 3
    assert native.library().risa_last_error() == b""


def test_lane_word_size_query_rules():
    """risa_mask_lanes_bytes is a host function: the size of the lane words of a boolean mask
    that enough heads share, 0 wherever the attention kernel reads the mask itself."""
    lib = native.library()
    BOOL, F32 = 3, 0

    def size(dtype=BOOL, head_dim=128, cta_k=64, stride_q=4608, stride_k=1, batch=2, heads=24,
             mask_batch=2, mask_heads=1, q_len=4096, k_len=4608):
        return lib.risa_mask_lanes_bytes(dtype, head_dim, cta_k, stride_q, stride_k, batch, heads,
                                         mask_batch, mask_heads, q_len, k_len)

    # [mask batch, mask heads, blocks of 32 queries padded to 128, 64-key tiles, 32 words] x 8 bytes,
    # then one 32-bit class per (block of 32 queries, tile), then per plane and block of 128
    # queries a tile list (tiles + 1 entries of 32 bits); every section a whole number of 8 bytes
    def expected(planes, q_len, k_len):
        waves, tiles = -(-q_len // 128) * 4, -(-k_len // 64)
        round8 = lambda n: -(-n // 8) * 8
        return planes * waves * tiles * 32 * 8 + round8(planes * waves * tiles * 4) + round8(planes * (waves // 4) * (tiles + 1) * 4)

    assert size() == expected(2, 4096, 4608)
    assert size(q_len=4000, k_len=4600) == expected(2, 4000, 4600)  # ragged extents round up
    assert size(batch=1, heads=24, mask_batch=1, q_len=1500, k_len=100) == expected(1, 1500, 100)
    assert size(head_dim=64) == size()
    assert size(dtype=F32) == 0            # values, not decisions
    assert size(cta_k=128) == 0            # query-dependent masks run 64-key tiles
    assert size(head_dim=256) == 0         # the sixteen-query kernel has another score layout
    assert size(stride_q=0) == 0           # key-only masks have their bias row
    assert size(stride_k=2) == 0
    assert size(mask_heads=24) == 0        # a plane per head: nobody to share with
    assert size(heads=7) == 0 and size(heads=8) > 0  # eight (batch, head) pairs per mask plane
    assert size(batch=1, heads=8, mask_batch=1, q_len=4096) == 0   # 256 workgroups: a small launch
    assert size(batch=1, heads=8, mask_batch=1, q_len=4224) > 0
    assert size(q_len=0) == 0


def test_host_only_entry_points():
    assert native.unpack_order() == layout.position_to_token()
    assert sorted(native.unpack_order()) == list(range(32))
    lib = native.library()
    assert lib.risa_selector_workspace_size(4096) == 0
    small = lib.risa_quantize_v_workspace_bytes(1, 4, 32768, 128, 0)
    large = lib.risa_quantize_v_workspace_bytes(1, 4, 32768, 128, 1)
    assert 0 < small < large
    # rejected calls report through risa_last_error and launch nothing
    assert lib.risa_quantize_qk(None, None, None, None, None, None, 1, 1, 1, 1, 1, 96, 64,
                                0, 0, 0, 0, 0, 0, 2, None, None, None) != 0
    assert b"head_dim" in lib.risa_last_error()
    with pytest.raises(RuntimeError, match="head_dim"):
        native.check(1)


def test_availability_gate_requires_rocm_gfx950():
    assert not risa.int8_attention_is_available("cpu")

    class Props:
        gcnArchName = "gfx950:sramecc+:xnack-"

    with patch.object(torch.version, "hip", "7.0"), patch.object(torch.cuda, "is_available", return_value=True), \
            patch.object(torch.cuda, "get_device_properties", return_value=Props()):
        assert native.is_available()
        Props.gcnArchName = "gfx942:sramecc+:xnack-"
        assert not native.is_available()
    with patch.object(torch.version, "hip", None):
        assert not native.is_available()


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    monkeypatch.setenv("RISA_HIP_LIBRARY", str(tmp_path / "absent.so"))
    monkeypatch.setattr(native, "_LIBRARY", None)
    monkeypatch.setattr(native, "_LOAD_ERROR", None)
    with pytest.raises(RuntimeError, match="not available"):
        native.library()
    assert not native.is_available()
    monkeypatch.setattr(native, "_LOAD_ERROR", None)


def test_public_names_match_reference_surface():
    assert set(risa.__all__) == {
        "KVPermutation", "prepare_kv_permutation", "PrequantizedInt8Attention", "RetainedMassPattern",
        "build_retained_mass_pattern", "construct_sparse_int8_attention",
        "construct_sparse_int8_attention_from_prequantized", "int8_attention",
        "int8_attention_from_prequantized", "int8_attention_is_available", "measure_pattern_recall",
        "prequantize_int8_attention", "sparse_int8_attention",
    }
    fields = [f for f in types.PrequantizedInt8Attention.__dataclass_fields__]
    assert fields[:16] == ["q", "k", "v", "q_scale", "k_scale", "v_scale", "v_center", "original_head_dim",
                           "input_dtype", "attention_scale", "cta_k", "attn_mask", "v_quantization",
                           "is_causal", "lse_shift", "kv_permuted"]


def test_tile_policy_and_constants():
    assert policy.select_key_block_size(128, 1025, has_mask=False) == 128
    assert policy.select_key_block_size(128, 1024, has_mask=False) == 64
    assert policy.select_key_block_size(256, 5000, has_mask=True) == 64
    assert policy.select_key_block_size(64, 5000, has_mask=False) == 64
    assert policy.pad_key_length(1153, 128) == 1280 and policy.pad_key_length(64) == 64
    assert policy.MIN_PATTERN_SPARSITY == 0.05 and policy.QUERY_BLOCK_SIZE == 128
    assert policy.DTYPE_CODES == {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def test_invalid_v_mode_and_input_errors():
    q = torch.empty(1)
    with pytest.raises(ValueError, match="v_quantization"):
        risa.int8_attention(q, q, q, v_quantization="invalid")
    x = torch.zeros(1, 2, 3, 64)
    with pytest.raises(ValueError, match="shape"):
        policy.validate_inputs(x[0], x, x, None)
    with pytest.raises(TypeError, match="float32, float16, or bfloat16"):
        policy.validate_inputs(x.double(), x.double(), x.double(), None)
    with pytest.raises(TypeError, match="same dtype"):
        policy.validate_inputs(x, x.half(), x, None)
    with pytest.raises(ValueError, match="same CUDA device"):
        policy.validate_inputs(x, x, x, None)  # CPU tensors


def test_validation_after_device_gate():
    x = torch.zeros(1, 4, 3, 64)

    class Fake(torch.Tensor):
        is_cuda = True

    def cuda_like(t):
        return t.as_subclass(Fake)

    with patch.object(policy, "is_available", return_value=True):
        q = cuda_like(x)
        with pytest.raises(ValueError, match="divisible"):
            policy.validate_inputs(q, cuda_like(torch.zeros(1, 3, 3, 64)), cuda_like(torch.zeros(1, 3, 3, 64)), None)
        with pytest.raises(ValueError, match=r"head_dim must be in \[1, 256\]"):
            big = cuda_like(torch.zeros(1, 1, 2, 300))
            policy.validate_inputs(big, big, big, None)
        with pytest.raises(TypeError, match="attn_mask must be bool"):
            policy.validate_inputs(q, q, q, torch.zeros(3, 3, dtype=torch.int32))
        with pytest.raises(ValueError, match="broadcastable"):
            policy.validate_inputs(q, q, q, torch.zeros(5, 5, dtype=torch.bool))
        mask = policy.validate_inputs(q, q, q, torch.ones(1, 1, 1, 3, dtype=torch.bool))
        assert mask.shape == (1, 4, 3, 3) and mask.stride(-2) == 0
    with patch.object(policy, "is_available", return_value=False):
        with pytest.raises(RuntimeError, match="gfx950"):
            policy.validate_inputs(cuda_like(x), cuda_like(x), cuda_like(x), None)


def test_custom_ops_propagate_causal_and_quantization():
    q = torch.randn(1, 2, 3, 64)
    for mode in ("midpoint_affine", "absmax"):
        for causal in (False, True):
            for mask in (None, torch.ones(3, 3, dtype=torch.bool)):
                with patch.object(dense, "execute_dense_attention", return_value=q.clone()) as launch:
                    risa.int8_attention(q, q, q, attn_mask=mask, is_causal=causal, v_quantization=mode)
                assert launch.call_args.kwargs["is_causal"] == causal
                assert launch.call_args.kwargs["use_midpoint_affine"] == (mode == "midpoint_affine")
                assert (launch.call_args.kwargs["attn_mask"] is None) == (mask is None)


def test_fake_tensor_shapes():
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        q = torch.empty(1, 2, 17, 64, device="cuda")
        for mode in ("midpoint_affine", "absmax"):
            result = risa.int8_attention(q, q, q, is_causal=True, v_quantization=mode)
            assert result.shape == q.shape
            masked = risa.int8_attention(q, q, q, attn_mask=torch.empty(17, 17, device="cuda", dtype=torch.bool))
            assert masked.shape == q.shape


def test_operator_is_recorded_whenever_the_dispatcher_is_watched():
    """Plain eager tensors skip the operator dispatch; under make_fx(real), a
    TorchDispatchMode or torch.jit.trace the call must go through
    risa_attention::int8_attention[_masked] (reference src/risa_attention/dense.py:123-146
    always dispatches through them), or the recorded graph would miss the kernel."""
    from torch.fx.experimental.proxy_tensor import make_fx
    from torch.utils._python_dispatch import TorchDispatchMode

    q = torch.randn(1, 2, 3, 64)
    mask = torch.ones(3, 3, dtype=torch.bool)
    with patch.object(dense, "execute_dense_attention", side_effect=lambda q, *a, **k: q.clone()):
        # eager: no operator involved
        seen = []

        class Recorder(TorchDispatchMode):
            def __torch_dispatch__(self, func, types, args=(), kwargs=None):
                seen.append(str(func))
                return func(*args, **(kwargs or {}))

        assert dense._plain_eager(q, q, q, None)
        with Recorder():
            assert not dense._plain_eager(q, q, q, None)
            risa.int8_attention(q, q, q)
            risa.int8_attention(q, q, q, attn_mask=mask)
        assert any("risa_attention.int8_attention.default" in name for name in seen)
        assert any("risa_attention.int8_attention_masked.default" in name for name in seen)

        graph = make_fx(lambda a: risa.int8_attention(a, a, a) + 1, tracing_mode="real")(q)
        targets = [str(node.target) for node in graph.graph.nodes if node.op == "call_function"]
        assert any("risa_attention.int8_attention" in name for name in targets), targets
        masked = make_fx(lambda a, m: risa.int8_attention(a, a, a, attn_mask=m), tracing_mode="real")(q, mask)
        targets = [str(node.target) for node in masked.graph.nodes if node.op == "call_function"]
        assert any("risa_attention.int8_attention_masked" in name for name in targets), targets

        traced = torch.jit.trace(lambda a: risa.int8_attention(a, a, a), (q,), check_trace=False)
        assert "risa_attention::int8_attention" in str(traced.graph)


def test_mask_signature_and_score_mask():
    mask = torch.ones(1, 1, 3, 5, dtype=torch.bool)
    before = policy.mask_signature(mask)
    mask[..., 0] = False
    assert before != policy.mask_signature(mask)
    assert policy.mask_signature(None) is None
    scores = policy.apply_score_mask(torch.zeros(1, 1, 3, 5), mask, True, 0)
    assert torch.isneginf(scores[..., 0, :]).all()
    assert torch.isneginf(scores[..., 1, 2:]).all()
    assert scores[0, 0, 1, 1] == 0
    shifted = policy.apply_score_mask(torch.zeros(1, 1, 2, 5), torch.full((1, 1, 3, 5), 2.0), False, 1)
    assert (shifted == 2).all()


def test_pattern_properties_and_prequantized_checks():
    pattern = types.RetainedMassPattern(
        row_offsets=torch.tensor([0, 1, 3], dtype=torch.int32), block_indices=torch.tensor([0, 0, 1], dtype=torch.int32),
        batch_size=1, q_heads=1, q_length=200, kv_length=130, query_block_size=128, key_block_size=64,
        attention_scale=0.1, retained_mass_target=0.9, measured_retained_mass=0.95)
    assert pattern.coverage == pytest.approx(3 / 6) and pattern.sparsity == pytest.approx(0.5)
    assert pattern.index_bytes == 6 * 4
    with pytest.raises(TypeError, match="prequantize_int8_attention"):
        risa.int8_attention_from_prequantized(object())
    packed = types.PrequantizedInt8Attention(*([torch.zeros(1)] * 7), 64, torch.float16, 0.1, 64, None)
    with pytest.raises(ValueError, match="output_layout"):
        risa.int8_attention_from_prequantized(packed, output_layout="dnh")
    with pytest.raises(ValueError, match="return_lse=True"):
        risa.int8_attention_from_prequantized(packed, return_lse=True)
    with pytest.raises(ValueError, match="CUDA device"):
        risa.int8_attention_from_prequantized(packed)
    with pytest.raises(ValueError, match="theta"):
        risa.construct_sparse_int8_attention_from_prequantized(packed, theta=0.0)
    with pytest.raises(TypeError, match="prequantize_int8_attention"):
        risa.construct_sparse_int8_attention_from_prequantized(object(), theta=0.5)


def test_pattern_compatibility_checks():
    q = torch.zeros(1, 2, 200, 64, dtype=torch.int8)
    packed = types.PrequantizedInt8Attention(q, torch.zeros(1, 1, 130, 64, dtype=torch.int8), *([torch.zeros(1)] * 5),
                                             64, torch.float16, 0.125, 64, None)
    good = dict(row_offsets=torch.zeros(5, dtype=torch.int32), block_indices=torch.zeros(4, dtype=torch.int32),
                batch_size=1, q_heads=2, q_length=200, kv_length=130, query_block_size=128, key_block_size=64,
                attention_scale=0.125, retained_mass_target=0.9, measured_retained_mass=0.9)
    attend.check_pattern(packed, types.RetainedMassPattern(**good))
    with pytest.raises(ValueError, match="is_causal"):
        attend.check_pattern(packed, types.RetainedMassPattern(**{**good, "is_causal": True}))
    with pytest.raises(ValueError, match="metadata"):
        attend.check_pattern(packed, types.RetainedMassPattern(**{**good, "key_block_size": 128}))
    with pytest.raises(ValueError, match="same scale"):
        attend.check_pattern(packed, types.RetainedMassPattern(**{**good, "attention_scale": 0.126}))
    with pytest.raises(ValueError, match="mask has changed"):
        attend.check_pattern(packed, types.RetainedMassPattern(**{**good, "mask_signature": (1,)}))
    with pytest.raises(TypeError, match="contiguous int32"):
        attend.check_pattern(packed, types.RetainedMassPattern(**{**good, "row_offsets": torch.zeros(5, dtype=torch.int64)}))
    with pytest.raises(TypeError, match="build_retained_mass_pattern"):
        attend.check_pattern(packed, object())


def test_packed_value_layout_round_trip():
    logical = torch.arange(2 * 96, dtype=torch.int8).reshape(2, 96)
    packed = layout.pack_values(logical)
    assert torch.equal(layout.unpack_values(packed), logical)
    order = layout.position_to_token()
    assert order[:8] == [0, 1, 2, 3, 8, 9, 10, 11] and order[16:20] == [4, 5, 6, 7]
    assert torch.equal(packed[0, :32], logical[0, order])


def test_fp32_pattern_builder_and_recall_on_cpu():
    g = torch.Generator().manual_seed(0)
    centroids = torch.randn(4, 64, generator=g) * 3
    tokens = centroids.repeat_interleave(64, 0)[None, None] + torch.randn(1, 2, 256, 64, generator=g) * 0.3
    q = k = tokens.contiguous()
    pattern = fp32_patterns.build_retained_mass_pattern(q, k, theta=0.9)
    assert pattern.key_block_size == 64 and pattern.query_block_size == 128
    assert pattern.row_offsets.tolist()[0] == 0 and pattern.row_offsets[-1] == pattern.block_indices.numel()
    assert 0 < pattern.coverage < 1
    assert pattern.measured_retained_mass >= 0.9
    recall = fp32_patterns.measure_pattern_recall(q, k, pattern)
    assert recall == pytest.approx(pattern.measured_retained_mass, abs=1e-5)
    dense_pattern = fp32_patterns.build_retained_mass_pattern(q, k, theta=1.0)
    assert fp32_patterns.measure_pattern_recall(q, k, dense_pattern) == pytest.approx(1.0, abs=1e-6)
    with pytest.raises(ValueError, match="theta"):
        fp32_patterns.build_retained_mass_pattern(q, k, theta=1.5)
    with pytest.raises(ValueError, match="pattern mask has changed"):
        fp32_patterns.measure_pattern_recall(q, k, pattern, attn_mask=torch.ones(256, 256, dtype=torch.bool))


def test_bench_rejects_more_than_one_gpu():
    import subprocess
    import sys

    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert done.returncode != 0 and "one MI355X" in done.stderr


def test_bench_paired_timing_rotates_and_reverses_positions():
    """bench.py's timing protocol (reference benchmarks/common.py:184-220): after the warm-ups
    every sample runs all methods, in the name order rotated by the sample index and reversed
    on every other complete rotation."""
    import importlib.util
    import types as pytypes

    spec = importlib.util.spec_from_file_location("bench_module", ROOT / "bench.py")
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)

    class Event:
        clock = 0.0

        def __init__(self, enable_timing=True):
            self.at = None

        def record(self, stream=None):
            Event.clock += 1.0
            self.at = Event.clock

        def synchronize(self):
            pass

        def elapsed_time(self, other):
            return other.at - self.at

    fake = pytypes.SimpleNamespace(cuda=pytypes.SimpleNamespace(
        current_stream=lambda: None, synchronize=lambda: None, Event=Event))
    calls = []
    methods = {name: (lambda name=name: calls.append(name)) for name in "abc"}
    stats = bench.measure_methods(fake, methods, samples=6, calls_per_sample=2, warmup=1)
    assert calls[:3] == ["a", "b", "c"]  # warm-ups
    order = calls[3::2]
    assert order == list("abc" "bca" "cab" "cba" "bac" "acb")
    assert all(len(stats[name]["samples_ms"]) == 6 and stats[name]["median_ms"] == 0.5 for name in "abc")
    assert bench.percentile([1.0, 2.0, 3.0, 4.0], 0.5) == 2.5
    # per-seed records in the reference's result schema -> median of the per-seed medians, mean accuracy
    def record(seed, median, nrmse, stage="dense", sparse=None):
        return {"case": "B1_Hq16_Hkv4_Lq512_Lk512_D128", "shape": {}, "seed": seed, "layout": "hnd",
                "qk_distribution": "normal", "value_distribution": "normal", "implementation": "risaattention_amd",
                "v_quantization": "absmax", "stage": stage,
                "timing": {"median_ms": median, "p10_ms": median - 0.001, "p90_ms": median + 0.001},
                "accuracy": {"nrmse": nrmse, "rmse": 1e-4, "sqnr_db": 36.0, "mae": 1e-4, "max_abs": 1e-3,
                             "max_channel_bias": 1e-4},
                "memory": {"peak_incremental_mib": 10.0 + seed}, "sparse": sparse}

    records = [record(0, 0.030, 0.0150), record(1, 0.025, 0.0140), record(2, 0.026, 0.0145)]
    records += [record(seed, 0.020, 0.02, "reuse", {"coverage": 0.5, "pattern_index_mib": 1.0,
                                                    "exact_construction_recall": 0.99, "current_recall": 0.98})
                for seed in (0, 1)]
    rows = bench.summarize_records(records)
    dense_row = next(row for row in rows if row["stage"] == "dense")
    assert dense_row["seed_count"] == 3 and dense_row["median_ms"] == 0.026
    assert dense_row["nrmse"] == pytest.approx(0.0145) and dense_row["peak_incremental_mib"] == 11.0
    assert dense_row["coverage"] is None
    reuse_row = next(row for row in rows if row["stage"] == "reuse")
    assert reuse_row["coverage"] == 0.5 and reuse_row["current_recall"] == 0.98
    import tempfile

    with tempfile.TemporaryDirectory() as folder:
        csv_path = Path(folder) / "summary.csv"
        report = bench.render_report({
            "suite": "sweep", "measured_at_utc": "now", "reference": "fp32",
            "environment": {"gpu": "MI355X", "arch": "gfx950"},
            "config": {"timing_order": "rotate-and-reverse", "seeds": [0, 1, 2], "samples": 10},
            "results": records}, csv_path)
        assert "| B1_Hq16_Hkv4_Lq512_Lk512_D128 | absmax | dense | 3 | 0.026 |" in report
        header, first, *_ = csv_path.read_text().splitlines()
        assert header.startswith("case,layout,qk_distribution") and "0.026" in first


def _bench_module():
    import importlib.util

    spec = importlib.util.spec_from_file_location("bench_module", ROOT / "bench.py")
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    return bench


def _bench_record(length, seed, median_ms, stage="dense", mode="absmax", sqnr=36.0, **extra):
    record = {"case": f"B1_Hq16_Hkv4_Lq{length}_Lk{length}_D128",
              "shape": {"batch": 1, "q_heads": 16, "kv_heads": 4, "q_len": length, "k_len": length, "head_dim": 128},
              "seed": seed, "layout": "hnd", "qk_distribution": "normal", "value_distribution": "normal",
              "implementation": "risaattention_amd", "v_quantization": mode, "stage": stage,
              "timing": {"median_ms": median_ms, "p10_ms": median_ms, "p90_ms": median_ms},
              "accuracy": None if sqnr is None else {"nrmse": 10 ** (-sqnr / 20), "rmse": 1e-4, "sqnr_db": sqnr, "mae": 1e-4,
                                                     "max_abs": 1e-3, "max_channel_bias": 1e-4},
              "memory": None, "sparse": None}
    record.update(extra)
    return record


def test_bench_mask_tile_benchmark_inputs_and_rows():
    """The broadcast-mask benchmark (reference benchmarks/masks.py:40-75): hidden tiles are taken
    from the order evens-then-odds, so they interleave with visible ones; the rows report every
    method against the same method with nothing hidden."""
    import torch

    bench = _bench_module()
    assert bench.empty_key_tiles(8, 0.0) == []
    assert bench.empty_key_tiles(8, 0.25) == [0, 2]
    assert bench.empty_key_tiles(8, 0.5) == [0, 2, 4, 6]
    assert bench.empty_key_tiles(8, 0.75) == [0, 1, 2, 3, 4, 6]  # all evens, then odds 1 and 3
    assert bench.empty_key_tiles(5, 1.0) == [0, 1, 2, 3, 4]
    mask = bench.interleaved_key_mask(torch, 2048, 128, 0.25, "bool", "cpu")  # 16 tiles of 128 keys
    assert mask.shape == (1, 1, 1, 2048) and mask.dtype == torch.bool
    hidden = (~mask).reshape(16, 128)
    assert hidden.all(1).tolist() == [tile in (0, 2, 4, 6) for tile in range(16)] and not hidden[1].any()
    short = bench.interleaved_key_mask(torch, 1024, 128, 0.5, "fp32", "cpu")  # 64-key tiles up to 1024 keys
    assert short.dtype == torch.float32 and torch.isneginf(short).sum().item() == 512
    assert torch.isneginf(short.reshape(16, 64)).all(1).tolist() == [tile % 2 == 0 for tile in range(16)]
    assert (short[torch.isfinite(short)] == 0).all()

    records = []
    for fraction, ms in ((0.0, 0.100), (0.5, 0.060)):
        for seed, jitter in ((0, 0.0), (1, 0.002), (2, -0.002)):
            for build, slower in (("after", 1.0), ("before", 1.5)):
                records.append(_bench_record(4096, seed, (ms + jitter) * slower, stage=f"{build}/mask_bool_empty_{fraction}",
                                             mask_empty_fraction=fraction, mask_dtype="bool", build=build,
                                             native_comparison={"bitwise_equal": seed != 2, "max_abs_difference": 0.0}))
    ops = bench.dense_equivalent_ops(1, 16, 4096, 4096, 128)
    rows = {(row["build"], row["empty_fraction"]): row for row in bench.mask_tile_rows(records, ops)}
    assert rows[("after", 0.5)]["ms"] == 0.06 and rows[("after", 0.5)]["vs_nothing_hidden"] == 0.6
    assert rows[("before", 0.0)]["ms"] == pytest.approx(0.15) and rows[("before", 0.5)]["vs_nothing_hidden"] == 0.6
    assert rows[("after", 0.0)]["tops"] == pytest.approx(ops / 0.1e-3 / 1e12, rel=1e-3)
    assert rows[("after", 0.0)]["bitwise_equal_to_baseline"] is False  # one seed differed


def test_bench_scaling_plot_inputs_and_figure(tmp_path):
    """Dense-equivalent TOPS over N for the plot (reference benchmarks/plot_scaling.py:66-75):
    4*B*Hq*Lq*Lk*D operations over the median of the per-seed medians, whatever a method skips."""
    bench = _bench_module()
    records = []
    for length, ms in ((1024, 0.02), (4096, 0.1)):
        for seed, jitter in ((0, 0.0), (1, 0.01), (2, -0.005)):
            records.append(_bench_record(length, seed, ms + jitter, sqnr=36.0 + seed))
            records.append(_bench_record(length, seed, (ms + jitter) / 2, stage="reuse", sqnr=None))
    records.append(_bench_record(2048, 0, 1.0) | {"shape": {"batch": 1, "q_heads": 16, "kv_heads": 4, "q_len": 2048,
                                                            "k_len": 4096, "head_dim": 128}})  # unequal lengths: left out
    series = bench.scaling_series(records)
    assert set(series) == {"dense/absmax", "reuse/absmax"}
    dense = series["dense/absmax"]
    assert [point["length"] for point in dense] == [1024, 4096]
    assert dense[0]["tops"] == pytest.approx(4 * 16 * 1024 * 1024 * 128 / 0.02e-3 / 1e12)
    assert dense[1]["sqnr_db"] == pytest.approx(37.0)
    assert series["reuse/absmax"][1]["tops"] == pytest.approx(2 * dense[1]["tops"]) and series["reuse/absmax"][1]["sqnr_db"] is None
    target = tmp_path / "figures" / "scaling.png"
    bench.plot_scaling(series, target, "sweep - MI355X (gfx950)")
    assert target.read_bytes()[:8] == b"\x89PNG\r\n\x1a\n" and target.stat().st_size > 10_000


def test_bench_profile_range_names():
    """One range per V mode and pass, named like the reference's (benchmarks/profile_operators.py:53-61)."""
    bench = _bench_module()
    assert bench.profile_range_names("dense", ("absmax", "midpoint_affine")) == ["risa/dense/absmax", "risa/dense/midpoint_affine"]
    assert bench.profile_range_names("attend", ("absmax",)) == ["risa/attend/absmax"]


def test_library_swap_routes_calls_and_restores():
    """native.using_library: calls inside the block reach the other build, the cached workspace
    sizes are dropped on both edges, and the in-tree library is back afterwards (also after an error)."""
    from risaattention_amd import attend

    own = native.library()
    other = native.load_library(native.library_path())  # a second handle on the same file
    assert other.risa_abi_version() == own.risa_abi_version()

    class Recorder:
        def __getattr__(self, name):
            return getattr(other, name)

        def risa_abi_version(self):
            return -7

    attend.sdpa_workspace_bytes(1, 2, 64, 2, 64, 128, 64, 0, -1, 0, 1, 1, 1)
    assert attend.sdpa_workspace_bytes.cache_info().currsize >= 1
    with native.using_library(Recorder()):
        assert attend.sdpa_workspace_bytes.cache_info().currsize == 0
        assert native.library().risa_abi_version() == -7
    assert native.library() is own and attend.sdpa_workspace_bytes.cache_info().currsize == 0
    with pytest.raises(KeyError):
        with native.using_library(Recorder()):
            raise KeyError("inside")
    assert native.library() is own
    with pytest.raises(OSError):
        native.load_library(ROOT / "no_such_library.so")
