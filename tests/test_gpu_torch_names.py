"""The reference's Python-side names (torch.cswapinit_ / cswapinit / cswapsetratio / cswappre /
cswappost) on stock PyTorch-ROCm: models written the way the reference's model files are
(CIFAR10/models/vgg.py:21-46: every layer between a cswappre and a cswappost of its input)
train with the same gradients as the plain model."""
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch


def make_model(torch, kind, codes):
    """kind: "cnn" (conv relu conv relu pool, twice, then a classifier, as the reference's VGG) or "mlp"
    (Linear/ReLU, whose backward is bit-reproducible); codes: the policy code the reference's layer_maker
    would pass for each layer of `features`, or None for the plain model."""

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            torch.manual_seed(0)
            layers = []
            if kind == "cnn":
                c = 3
                for v in (32, 32, "M", 64, 64, "M"):
                    if v == "M":
                        layers.append(torch.nn.MaxPool2d(2))
                    else:
                        layers += [torch.nn.Conv2d(c, v, 3, padding=1), torch.nn.ReLU()]
                        c = v
                self.classifier = torch.nn.Linear(64 * 16 * 16, 10)
            else:
                for a, b in ((512, 1024), (1024, 1024), (1024, 1024)):
                    layers += [torch.nn.Linear(a, b), torch.nn.ReLU()]
                self.classifier = torch.nn.Linear(1024, 16)
            self.features = torch.nn.ModuleList(layers)

        def forward(self, out):
            if codes is not None:
                torch.cswapinit()
            for i, layer in enumerate(self.features):
                out = self.layer_maker(layer, out, 0 if codes is None else codes[i])
            pre = out
            if codes is not None:
                torch.cswappre(pre, 0)
            out = pre.view(pre.size(0), -1)
            if codes is not None:
                torch.cswappost(pre, out, 0)
            return self.layer_maker(self.classifier, out, 0 if codes is None else codes[-1])

        def layer_maker(self, layer, input, type):  # noqa: A002
            pre = input
            if codes is not None:
                torch.cswappre(pre, type)
            out = layer(pre)
            if codes is not None:
                torch.cswappost(pre, out, type)
            return out

    return Net().cuda()


def run(torch, net, x):
    net.zero_grad(set_to_none=True)
    loss = net(x).square().mean()
    loss.backward()
    torch.cuda.synchronize()
    return float(loss.detach()), [p.grad.clone() for p in net.parameters()]


def test_lossless_codes_leave_the_gradients_bit_identical(torch_cuda):
    torch = torch_cuda
    from cswap_amd import torch_names as names

    x = torch.randn(2048, 512, device="cuda")
    loss0, g0 = run(torch, make_model(torch, "mlp", None), x)
    loss0b, g0b = run(torch, make_model(torch, "mlp", None), x)
    assert loss0 == loss0b and all(torch.equal(a, b) for a, b in zip(g0, g0b)), "baseline is not deterministic"
    names.install()
    try:
        torch.cswapinit_(pinned_bytes=256 << 20, device_bytes=128 << 20)
        # features: Linear ReLU Linear ReLU Linear ReLU, then the classifier; a layer's code is the policy of its
        # INPUT.  Autograd keeps the three ReLU outputs (each for the ReLU node and for the Linear after it);
        # the batch has no grad_fn and nobody keeps the inputs of the ReLUs.
        for codes, by in (([2, 2, 2, 2, 2, 2, 2], {"raw": 3}), ([0, 0, 3, 0, 3, 0, 3], {"zvc": 3}),
                          ([3, 3, 2, 3, 3, 3, 2], {"raw": 2, "zvc": 1})):
            for _ in range(2):                               # two iterations: cswapinit() ends the one before
                loss1, g1 = run(torch, make_model(torch, "mlp", codes), x)
                st = names.stats()
                assert st["swapped"] == 3 and st["by_policy"] == by, (codes, st)
                assert st["shared"] == 3                     # one swap for the two nodes that keep a ReLU output
                assert loss1 == loss0 and all(torch.equal(a, b) for a, b in zip(g0, g1)), codes
        # code 0 everywhere: nothing goes out
        loss2, g2 = run(torch, make_model(torch, "mlp", [0] * 7), x)
        assert names.stats().get("swapped", 0) == 0 and names.stats()["held"] >= 3
        assert loss2 == loss0 and all(torch.equal(a, b) for a, b in zip(g0, g2))
        # no autograd, no swapping
        with torch.no_grad():
            make_model(torch, "mlp", [2] * 7)(x)
        assert names.stats().get("swapped", 0) == 0
        with pytest.raises(ValueError):
            torch.cswappre(x, 5)
    finally:
        names.cswapclose()
        names.uninstall()
    assert not hasattr(torch, "cswappre")


def test_a_model_written_like_the_references_vgg(torch_cuda):
    """ZVC for the ReLU outputs and ZFP for the pooled one, the assignment of the reference's own
    drivers (CSWAP+/vgg16-cifar10.cpp:177-178,393-397).  Convolution backward is not bit-reproducible
    run to run, so the comparison has a tolerance."""
    torch = torch_cuda
    from cswap_amd import torch_names as names

    x = torch.randn(64, 3, 64, 64, device="cuda")
    loss0, g0 = run(torch, make_model(torch, "cnn", None), x)

    def close(ga, gb, rtol):
        return all(torch.allclose(a, b, rtol=rtol, atol=rtol * float(a.abs().max())) for a, b in zip(ga, gb))

    names.install()
    try:
        torch.cswapinit_(pinned_bytes=512 << 20, device_bytes=256 << 20)
        torch.cswapsetratio(128)
        # features: conv relu conv relu pool conv relu conv relu pool, then the classifier.  What autograd
        # keeps, and so what can go out: the inputs of the second to fourth convolution and of the two pools
        # (four ReLU outputs and one pool output).
        lossless = [2, 2, 3, 2, 3, 2, 2, 3, 2, 3, 0]
        loss1, g1 = run(torch, make_model(torch, "cnn", lossless), x)
        st = names.stats()
        assert st["swapped"] == 5 and st["by_policy"] == {"raw": 1, "zvc": 4}, st
        assert st["shared"] >= 4 and st["bytes_out"] < st["bytes_in"]
        assert abs(loss1 - loss0) <= 1e-6 * abs(loss0) and close(g0, g1, 1e-4)

        # and the device memory does go: at the end of forward four of the five swapped tensors (109 MB in
        # all) have left the device, the last one is still there for backward to pick up
        def held_after_forward(codes):
            net = make_model(torch, "cnn", codes)
            torch.cuda.synchronize()
            base = torch.cuda.memory_allocated()
            loss = net(x).square().mean()
            torch.cuda.synchronize()
            held = torch.cuda.memory_allocated() - base
            loss.backward()
            return held

        assert held_after_forward(lossless) < held_after_forward(None) - (80 << 20)

        mixed = [0, 0, 3, 0, 3, 6, 0, 3, 0, 3, 0]
        loss2, g2 = run(torch, make_model(torch, "cnn", mixed), x)
        st2 = names.stats()
        assert st2["swapped"] == 5 and st2["by_policy"] == {"zfp": 1, "zvc": 4}, st2
        assert close(g0, g2, 0.05) and not close(g0, g2, 1e-5)

        # twice the rate: the pooled tensor's stream doubles, the result gets closer
        torch.cswapsetratio(256)
        loss3, g3 = run(torch, make_model(torch, "cnn", mixed), x)
        st3 = names.stats()
        pooled = 64 * 32 * 32 * 32 * 4
        assert st3["bytes_out"] - st2["bytes_out"] == pooled // 2 - pooled // 4, (st2, st3)
        err2 = sum(float((a - b).square().sum()) for a, b in zip(g0, g2))
        err3 = sum(float((a - b).square().sum()) for a, b in zip(g0, g3))
        assert err3 < err2 / 100

        # the selector (code -1, which the reference does not have) picks per tensor
        torch.cswapsetratio(128)
        loss5, g5 = run(torch, make_model(torch, "cnn", [-1] * 10 + [0]), x)
        st5 = names.stats()
        assert st5["swapped"] == 5 and st5["by_policy"].get("zvc", 0) >= 2, st5
        # (a ReLU output that the selector gives to ZFP comes back with its exact zeros as +-epsilon, which
        # flips entries of the ReLU mask in backward: the whole gradient stays aligned, single entries move)
        va, vb = torch.cat([g.flatten() for g in g0]), torch.cat([g.flatten() for g in g5])
        assert float(torch.nn.functional.cosine_similarity(va, vb, dim=0)) > 0.98
    finally:
        names.cswapclose()
        names.uninstall()


def test_rate_change_between_swap_out_and_swap_in(torch_cuda):
    """A tensor comes back with the rate it went out with, whatever setRatio was called with since."""
    torch = torch_cuda
    from cswap_amd import api, swap

    eng = swap.SwapEngine(pinned_bytes=128 << 20, device_bytes=128 << 20, maxbits=512)
    try:
        x = torch.randn(32, 16, 32, 32, device="cuda")
        t8 = eng.pre(x, swap.ZFP)
        eng.set_maxbits(1024)
        t16 = eng.pre(x, swap.ZFP)
        eng.post(t8)
        eng.post(t16)
        assert eng.info(t8).bytes_out * 2 == eng.info(t16).bytes_out == x.numel() * 2
        eng.set_maxbits(256)
        out8, out16 = torch.empty_like(x), torch.empty_like(x)
        eng.swap_in(t8, out8)
        eng.swap_in(t16, out16)
        torch.cuda.synchronize()
        for out, maxbits in ((out8, 512), (out16, 1024)):
            want = api.cuda_decompress(api.cuda_compress(x, maxbits), x.shape, maxbits)
            assert torch.equal(out.view(torch.int32), want.view(torch.int32))
        eng.release(t8)
        eng.release(t16)
        with pytest.raises(Exception):
            eng.set_maxbits(8)
    finally:
        eng.close()
