"""risa_quantize_v_noalloc (the entry point that allocates nothing: its scratch memory is an
array built into the library) against risa_quantize_v on the same inputs, through the C ABI:
two calls in a row, the second with a smaller input, every output bit-equal."""

import pytest
import torch

pytestmark = pytest.mark.gpu

NOALLOC_MAX_BYTES = 16 << 20


def _prepare_both(risa, v, mode, cta_k, permutation=None):
    from risaattention_amd import native
    from risaattention_amd.policy import DTYPE_CODES

    lib = native.library()
    batch, heads, length, dim = v.shape
    padded = -(-length // cta_k) * cta_k
    affine = int(mode == "midpoint_affine")
    stream = native.current_stream(v.device)
    code = DTYPE_CODES[v.dtype]

    def buffers():
        return (torch.full((batch * heads * dim, padded), 77, dtype=torch.int8, device="cuda"),
                torch.full((batch * heads * dim,), -1.0, device="cuda"),
                torch.full((batch * heads * dim,), -1.0, device="cuda"),
                torch.full((batch * heads, padded // cta_k, dim), -1, dtype=torch.int32, device="cuda"))

    expected = buffers()
    needed = lib.risa_quantize_v_workspace_bytes(batch, heads, length, dim, affine)
    workspace = torch.empty(max(1, needed), dtype=torch.uint8, device="cuda")
    native.check(lib.risa_quantize_v(
        v.data_ptr(), *(t.data_ptr() for t in expected), workspace.data_ptr(), workspace.numel(), batch, heads,
        length, dim, padded, cta_k, *v.stride()[:3], code, affine, native.pointer(permutation), stream))
    actual = buffers()
    status = lib.risa_quantize_v_noalloc(
        v.data_ptr(), *(t.data_ptr() for t in actual), batch, heads, length, dim, padded, cta_k,
        *v.stride()[:3], code, affine, native.pointer(permutation), stream)
    return status, needed, expected, actual


@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_noalloc_entry_point_matches_workspace_entry_point_twice(risa, mode):
    from risaattention_amd import native

    generator = torch.Generator(device="cuda").manual_seed(5)
    # first call: 8 heads x 9000 tokens (partial-range and residual-partial buffers in use);
    # second call: a smaller problem, which finds the first call's leftovers in the array
    shapes = [((1, 8, 9000, 128), torch.bfloat16, 128), ((2, 2, 700, 64), torch.float16, 64)]
    for shape, dtype, cta_k in shapes:
        v = (torch.randn(shape, generator=generator, device="cuda") * 2.0 + 0.75).to(dtype)
        status, needed, expected, actual = _prepare_both(risa, v, mode, cta_k)
        native.check(status)
        assert 0 < needed <= NOALLOC_MAX_BYTES
        torch.cuda.synchronize()
        for ours, theirs, name in zip(actual, expected, ("codes", "scale", "center", "tile_sum")):
            assert torch.equal(ours, theirs), (shape, name)
        assert not (actual[0] == 77).all()


def test_noalloc_entry_point_with_a_permutation_and_strided_values(risa):
    from risaattention_amd import native

    generator = torch.Generator(device="cuda").manual_seed(6)
    storage = torch.randn(1, 3000, 3, 2, 128, generator=generator, device="cuda").to(torch.float16)
    v = storage[:, :, 2].transpose(1, 2)  # [1, 2, 3000, 128], token-major storage
    order = torch.stack([torch.randperm(3000, generator=generator, device="cuda") for _ in range(2)])
    order = order.reshape(1, 2, 3000).to(torch.int32).contiguous()
    status, _, expected, actual = _prepare_both(risa, v, "midpoint_affine", 128, order)
    native.check(status)
    torch.cuda.synchronize()
    for ours, theirs in zip(actual, expected):
        assert torch.equal(ours, theirs)


@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_noalloc_entry_point_allocates_nothing_and_replays_from_a_graph(risa, mode):
    """What the entry point exists for: after its first call on a device it changes nothing in
    the device's free memory, and a call recorded into a HIP graph replays bit-equal to
    risa_quantize_v on whatever the input buffer holds at the time of the replay."""
    from risaattention_amd import native
    from risaattention_amd.policy import DTYPE_CODES

    lib = native.library()
    batch, heads, length, dim, cta_k = 1, 4, 5000, 128, 128
    padded = -(-length // cta_k) * cta_k
    affine = int(mode == "midpoint_affine")
    generator = torch.Generator(device="cuda").manual_seed(9)
    v = torch.randn(batch, heads, length, dim, generator=generator, device="cuda").to(torch.bfloat16)
    outputs = (torch.zeros(batch * heads * dim, padded, dtype=torch.int8, device="cuda"),
               torch.zeros(batch * heads * dim, device="cuda"), torch.zeros(batch * heads * dim, device="cuda"),
               torch.zeros(batch * heads, padded // cta_k, dim, dtype=torch.int32, device="cuda"))

    def call(stream):
        native.check(lib.risa_quantize_v_noalloc(
            v.data_ptr(), *(t.data_ptr() for t in outputs), batch, heads, length, dim, padded, cta_k,
            *v.stride()[:3], DTYPE_CODES[v.dtype], affine, None, stream))

    call(native.current_stream(v.device))  # resolves the array's address on this device
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    call(native.current_stream(v.device))
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call(side.cuda_stream)
    for step in range(3):
        # eager work and a synchronisation between the replays
        v.copy_((torch.randn(v.shape, generator=generator, device="cuda") * (step + 1) - 0.5 * step).to(v.dtype))
        for t in outputs:
            t.fill_(3)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        _, _, expected, _ = _prepare_both(risa, v, mode, cta_k)
        torch.cuda.synchronize()
        for ours, theirs, name in zip(outputs, expected, ("codes", "scale", "center", "tile_sum")):
            assert torch.equal(ours, theirs), (step, name)


def test_noalloc_entry_point_rejects_problems_beyond_its_array(risa):
    from risaattention_amd import native

    v = torch.zeros(1, 40, 32768, 128, dtype=torch.bfloat16, device="cuda")
    status, needed, _, _ = _prepare_both(risa, v, "midpoint_affine", 128)
    assert needed > NOALLOC_MAX_BYTES
    assert status != 0
    message = native.library().risa_last_error().decode()
    assert "built-in buffer" in message and str(needed) in message
    with pytest.raises(RuntimeError, match="risa_quantize_v with a caller-provided workspace"):
        native.check(status)
