"""dlp_ip_fwd_enqueue_no_alloc (the entry point that allocates nothing) against dlp_ip_fwd_enqueue, through the C ABI.

The two entry points launch the same kernel; only the home of the tile counters and K-slice partial sums differs
(the library's device array instead of a buffer the operator allocates), so the results must be equal bit for bit.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import gpu_util

    return gpu_util


def _tensors(rng, batch, inputs, outputs):
    x = rng.uniform(-1, 1, (batch, inputs)).astype(np.float32)
    w = (rng.standard_normal((outputs, inputs)) / np.sqrt(inputs)).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, outputs).astype(np.float32)
    return x, w, b


def _both(gpu, op, x, w, b, dtype=None):
    """(result of enqueue, result of enqueue_no_alloc) as numpy, outputs poisoned with NaN beforehand"""
    import torch

    dtype = dtype or torch.float32
    xd, wd, bd = gpu.dev(x).to(dtype), gpu.dev(w).to(dtype), gpu.dev(b)
    want = torch.full((x.shape[0], w.shape[0]), float("nan"), dtype=dtype, device="cuda:0")
    got = torch.full_like(want, float("nan"))
    op.enqueue(xd, wd, bd, want)
    torch.cuda.synchronize()
    op.enqueue_no_alloc(xd, wd, bd, got)
    torch.cuda.synchronize()
    return want.float().cpu().numpy(), got.float().cpu().numpy()


def test_two_calls_in_a_row_second_smaller(gpu, oracle_mod):
    import dlprimitives_amd as dlp

    rng = np.random.default_rng(11)
    inputs, outputs = 2048, 1000  # the classifier of ResNet-50: K is split, so counters and partial sums are in use
    op = dlp.IPForward.create(dlp.IPSettings(inputs, outputs, 128), True, "relu")
    for batch in (128, 40):  # the second call finds the first call's partial sums in the array
        x, w, b = _tensors(rng, batch, inputs, outputs)
        want, got = _both(gpu, op, x, w, b)
        assert not np.isnan(got).any()
        assert np.array_equal(got, want)
        np.testing.assert_allclose(got, oracle_mod.ip_forward(x, w, b, "relu"), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("bio", [(1, 512, 1000), (16, 25088, 96), (33, 4100, 31), (3, 1030, 70), (2, 1, 1), (16, 1024, 20000), (16, 2048, 16000)], ids=lambda v: "b%d_%dto%d" % v)
def test_shapes_equal_the_allocating_entry_point(gpu, bio):
    import dlprimitives_amd as dlp

    batch, inputs, outputs = bio
    rng = np.random.default_rng(batch + inputs)
    x, w, b = _tensors(rng, batch, inputs, outputs)
    op = dlp.IPForward.create(dlp.IPSettings(inputs, outputs, batch), True, "identity")
    want, got = _both(gpu, op, x, w, b)
    assert np.array_equal(got, want)


def test_bf16_and_back_to_back_calls_on_one_stream(gpu):
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA

    rng = np.random.default_rng(3)
    x, w, b = _tensors(rng, 128, 2048, 1000)
    op = dlp.IPForward.create(dlp.IPSettings(2048, 1000, 128, dtype=BFLOAT16_DATA), True, "identity")
    want, got = _both(gpu, op, x, w, b, torch.bfloat16)
    assert np.array_equal(got, want)
    # calls queued back to back share the array without a host wait in between: the stream orders them
    xd, wd, bd = gpu.dev(x).to(torch.bfloat16), gpu.dev(w).to(torch.bfloat16), gpu.dev(b)
    ys = [torch.full((128, 1000), float("nan"), dtype=torch.bfloat16, device="cuda:0") for _ in range(4)]
    for y in ys:
        op.enqueue_no_alloc(xd, wd, bd, y)
    torch.cuda.synchronize()
    for y in ys:
        assert np.array_equal(y.float().cpu().numpy(), want)


def test_sizes_beyond_the_array_are_rejected(gpu):
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import ValidationError

    # rows that do not start on 16-byte boundaries take the direct kernel, whose plan cuts K whatever the number of tiles:
    # 128 blocks of outputs x 5 chunks of batch rows = 640 tiles of 4 KiB x 2 K slices: 5 MiB of partial sums
    # (the streaming kernel keeps tiles x K slices within 1024, so its partial sums stay within 4 MiB: 16 x 1024 -> 20000 above)
    inputs, outputs, batch = 1026, 4096, 160
    op = dlp.IPForward.create(dlp.IPSettings(inputs, outputs, batch), False, "identity")
    x = torch.zeros((batch, inputs), device="cuda:0")
    w = torch.zeros((outputs, inputs), device="cuda:0")
    y = torch.zeros((batch, outputs), device="cuda:0")
    with pytest.raises(ValidationError, match="scratch"):
        op.enqueue_no_alloc(x, w, None, y)
    op.enqueue(x, w, None, y)  # the allocating entry point takes it
    torch.cuda.synchronize()


def test_recorded_into_a_hip_graph_and_replayed(gpu):
    """What the entry point is for: the call is recorded into a HIP graph (it allocates nothing and records no memset: its
    counters are cleared by a kernel) and the graph is replayed, with eager work and synchronizations between the replays and on
    inputs that change between them; every replay must equal dlp_ip_fwd_enqueue on the same inputs bit for bit."""
    import torch

    import dlprimitives_amd as dlp

    rng = np.random.default_rng(21)
    batch, inputs, outputs = 64, 2048, 1000
    op = dlp.IPForward.create(dlp.IPSettings(inputs, outputs, batch), True, "relu")
    x, w, b = _tensors(rng, batch, inputs, outputs)
    xd, wd, bd = gpu.dev(x), gpu.dev(w), gpu.dev(b)
    got = torch.full((batch, outputs), float("nan"), device="cuda:0")
    op.enqueue_no_alloc(xd, wd, bd, got)  # one eager call first (module load, the array's address)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            op.enqueue_no_alloc(xd, wd, bd, got)
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        xn = rng.uniform(-1, 1, x.shape).astype(np.float32)
        xd.copy_(torch.from_numpy(xn))  # the graph holds the pointer, not the values
        got.fill_(float("nan"))
        want = torch.full_like(got, float("nan"))
        op.enqueue(xd, wd, bd, want)  # eager work of the program's own between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), want.cpu().numpy()), "replay %d" % replay
