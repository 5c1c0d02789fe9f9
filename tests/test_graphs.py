"""Whole-network forward: ResNet-18 / ResNet-50 graphs through the C-ABI operators on the GPU
against the same graph run with the oracle operators on the CPU (fp32)."""
import numpy as np
import pytest

from dlprimitives_amd import graphs


def test_graph_shapes_and_conv_multiset():
    r18 = graphs.resnet18()
    assert sum(o["op"] == "conv" for o in r18) == 20 and sum(o["op"] == "add" for o in r18) == 8
    r50 = graphs.resnet50()
    assert sum(o["op"] == "conv" for o in r50) == 53 and sum(o["op"] == "add" for o in r50) == 16
    sh = graphs.infer_shapes(r50, (2, 3, 224, 224))
    assert sh["stem"] == (2, 64, 112, 112) and sh["pool"] == (2, 64, 56, 56) and sh["l4_2"] == (2, 2048, 7, 7) and sh["logits"] == (2, 1000)
    # conv flops per image: 3.627 GFLOP (ResNet-18 conv stack), 8.174 GFLOP (ResNet-50)
    def conv_gflop(ops, shapes):
        return sum(2.0 * np.prod(shapes[o["dst"]][1:]) * o["cin"] * o["k"] ** 2 for o in ops if o["op"] == "conv") / 1e9
    assert abs(conv_gflop(r18, graphs.infer_shapes(r18, (1, 3, 224, 224))) - 3.627) < 0.002
    assert abs(conv_gflop(r50, sh) - 8.174) < 0.01


def test_batchnorm_fold_closed_form():
    rng = np.random.default_rng(0)
    w = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    gamma, beta, mean, var = (rng.uniform(0.5, 1.5, 4).astype(np.float32) for _ in range(4))
    wf, bf = graphs.fold_batchnorm(w, gamma, beta, mean, var)
    x = rng.standard_normal((3, 3, 3)).astype(np.float32)
    for o in range(4):
        conv = float((w[o] * x).sum())
        bn = (conv - mean[o]) / np.sqrt(var[o] + 1e-5) * gamma[o] + beta[o]
        assert abs(float((wf[o] * x).sum()) + bf[o] - bn) < 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("fuse_residual", [False, True], ids=["sums_as_operators", "sums_in_epilogues"])
@pytest.mark.parametrize("net", ["resnet18", "resnet50"])
def test_full_forward_matches_oracle(oracle_mod, net, fuse_residual):
    import torch

    from graph_oracle import run_graph_on_oracle

    ops = getattr(graphs, net)()
    params = graphs.random_parameters(ops, seed=7)
    x = np.random.default_rng(1).uniform(-1, 1, (2, 3, 224, 224)).astype(np.float32)
    runner = graphs.GraphRunner(ops, params, x.shape, fuse_residual=fuse_residual, prepack=fuse_residual)  # (filters transformed once, or in every call)
    # ResNet-50's 16 sums all follow a 1x1 convolution; ResNet-18's follow 3x3 convolutions and stay operators
    assert len(runner.ops) == len(ops) - (16 if fuse_residual and net == "resnet50" else 0)
    got = runner.forward(torch.from_numpy(x).cuda())
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    want = run_graph_on_oracle(oracle_mod, ops, params, x)
    scale = np.abs(want).max()
    assert scale > 0.1
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4 * scale)
    # the second run reuses every operator and the shared workspace
    got2 = runner.forward().cpu().numpy()
    assert np.array_equal(got, got2)
