"""Seeded synthetic activation tensors for the benchmark configurations.

All generators are numpy ``Generator(PCG64(seed))`` based so that the CPU
checker, the golden-vector script and the GPU runs see the same bytes on every
machine.  Fields are returned in zfp order ``(nz, ny, nx)``: nx is the last
tensor dimension, ny the second to last and nz the product of the rest, x
fastest in memory (CSWAP+/zfp/zfp.h:143, CSWAP+/zfp/cuZFP.cu:372-375).
"""
from __future__ import annotations

import math

import numpy as np


def as_field(t: np.ndarray) -> np.ndarray:
    """View an activation tensor [..., H, W] as the 3-D zfp field (nz, ny, nx)."""
    t = np.ascontiguousarray(t, dtype=np.float32)
    return t.reshape(-1, t.shape[-2], t.shape[-1])


def field_dims(shape):
    """(nx, ny, nz) of the field an activation tensor of ``shape`` maps to.

    nx = last dim, ny = second to last, nz = product of the rest.  Tensors with
    fewer than three useful dimensions would leave nz (or ny) at 1 and pay for
    4x4x4 blocks that are mostly padding, so they are folded: a matrix [B, F]
    with B a multiple of 4 becomes (F, 4, B/4); a flat vector becomes 32x32 or
    4x4 rows when its length allows.  Any such view of contiguous memory is a
    valid field as long as both directions use the same one."""
    shape = [int(d) for d in shape]
    if len(shape) <= 1:
        n = shape[0] if shape else 1
        if n % 1024 == 0:
            return 32, 32, n // 1024
        if n % 16 == 0:
            return 4, 4, n // 16
        return n, 1, 1
    nx, ny = shape[-1], shape[-2]
    nz = int(np.prod(shape[:-2])) if len(shape) > 2 else 1
    if nz < 4 and ny >= 16 and ny % 4 == 0:
        nz, ny = nz * (ny // 4), 4
    return nx, ny, nz


# -- configuration 1: [64,64,32,32] PReLU(N(0,1)), slope 0.25, seed 0 ---------
def config1_field() -> np.ndarray:
    x = np.random.default_rng(0).standard_normal((4096, 32, 32), dtype=np.float32)
    return np.where(x > 0, x, np.float32(0.25) * x).astype(np.float32)


# -- configuration 2: ReLU(N(mu,1)) with a chosen fraction of zeros -----------
_MU = {30: 0.5244005127080409, 50: 0.0, 70: -0.5244005127080409, 90: -1.2815515655446004}


def config2_tensor(sparsity_pct: int = 50, shape=(128, 256, 16, 16), seed: int = 0) -> np.ndarray:
    mu = _MU[sparsity_pct]
    x = np.random.default_rng(seed).standard_normal(shape, dtype=np.float32) + np.float32(mu)
    return np.maximum(x, np.float32(0)).astype(np.float32)


# -- configuration 3: VGG-16-style stack, LeakyReLU(0.01) x per-channel scale -
CONFIG3_SHAPES = {
    "64x32x32": (64, 32, 32),
    "128x16x16": (128, 16, 16),
    "256x8x8": (256, 8, 8),
    "512x4x4": (512, 4, 4),
    "512x2x2": (512, 2, 2),
}


def config3_fields(batch: int = 128) -> dict:
    out = {}
    for name, (c, h, w) in CONFIG3_SHAPES.items():
        x = np.random.default_rng(0).standard_normal((batch, c, h, w), dtype=np.float32)
        x = np.where(x > 0, x, np.float32(0.01) * x).astype(np.float32)
        scale = np.random.default_rng(1).uniform(0.1, 4.0, size=c).astype(np.float32)
        x = x * scale[None, :, None, None]
        out[name] = as_field(x.astype(np.float32))
    return out


# -- configuration 4: VGG-16 activation schedule at 3x64x64 input -------------
def config4_schedule(batch: int = 128):
    """Swapped tensors of a VGG-16 forward pass (the inputs of conv2..conv13,
    CSWAP+/vgg16-cifar10.cpp:177-178,396-397) plus the dense conv/BN outputs of
    the same shapes.  Returns a list of dicts {id, kind, shape}; ``kind`` is
    'relu' (40-80 % zeros), 'pool' (2x2 max of such) or 'dense' (N(0,1))."""
    sched = []
    tid = 0
    c_prev, hw = 3, 64
    plan = [(64, 2), (128, 2), (256, 3), (512, 3), (512, 3)]
    for c, reps in plan:
        for _ in range(reps):
            sched.append({"id": tid, "kind": "dense", "shape": (batch, c, hw, hw)}); tid += 1  # conv
            sched.append({"id": tid, "kind": "dense", "shape": (batch, c, hw, hw)}); tid += 1  # bn
            sched.append({"id": tid, "kind": "relu", "shape": (batch, c, hw, hw)}); tid += 1   # relu
            c_prev = c
        hw //= 2
        sched.append({"id": tid, "kind": "pool", "shape": (batch, c_prev, hw, hw)}); tid += 1
    return sched


def config4_tensor(entry, seed: int = 0) -> np.ndarray:
    rng = np.random.default_rng(seed + 1000 * entry["id"])
    shape = entry["shape"]
    if entry["kind"] == "dense":
        return rng.standard_normal(shape, dtype=np.float32)
    zeros = rng.uniform(0.40, 0.80)
    if entry["kind"] == "relu":
        mu = -_ndtri(zeros)
        x = rng.standard_normal(shape, dtype=np.float32) + np.float32(mu)
        return np.maximum(x, np.float32(0)).astype(np.float32)
    # pool: 2x2 max of a ReLU tensor twice the size
    b, c, h, w = shape
    mu = -_ndtri(zeros)
    x = rng.standard_normal((b, c, 2 * h, 2 * w), dtype=np.float32) + np.float32(mu)
    x = np.maximum(x, np.float32(0))
    return x.reshape(b, c, h, 2, w, 2).max(axis=(3, 5)).astype(np.float32)


def _ndtri(p: float) -> float:
    """Inverse normal CDF (Acklam's rational approximation, |err| < 1.2e-9)."""
    a = [-3.969683028665376e+01, 2.209460984245205e+02, -2.759285104469687e+02,
         1.383577518672690e+02, -3.066479806614716e+01, 2.506628277459239e+00]
    b = [-5.447609879822406e+01, 1.615858368580409e+02, -1.556989798598866e+02,
         6.680131188771972e+01, -1.328068155288572e+01]
    c = [-7.784894002430293e-03, -3.223964580411365e-01, -2.400758277161838e+00,
         -2.549732539343734e+00, 4.374664141464968e+00, 2.938163982698783e+00]
    d = [7.784695709041462e-03, 3.224671290700398e-01, 2.445134137142996e+00,
         3.754408661907416e+00]
    if p < 0.02425:
        q = math.sqrt(-2 * math.log(p))
        return (((((c[0]*q+c[1])*q+c[2])*q+c[3])*q+c[4])*q+c[5]) / ((((d[0]*q+d[1])*q+d[2])*q+d[3])*q+1)
    if p > 1 - 0.02425:
        return -_ndtri(1 - p)
    q = p - 0.5
    r = q * q
    return (((((a[0]*r+a[1])*r+a[2])*r+a[3])*r+a[4])*r+a[5])*q / (((((b[0]*r+b[1])*r+b[2])*r+b[3])*r+b[4])*r+1)


# -- configuration 5: BERT-base-sized dense activations -----------------------
CONFIG5_SHAPES = {
    "hidden_gelu": (32, 512, 768),
    "ffn_gelu": (32, 512, 3072),
    "attn_softmax": (32, 12, 512, 512),
}


def config5_tensor_torch(name: str, device, seed: int = 0, batch: int | None = None):
    """Configuration-5 tensors are generated on the device with torch (the
    402 MB softmax tensor is too slow to make with numpy every run)."""
    import torch

    shape = list(CONFIG5_SHAPES[name])
    if batch is not None:
        shape[0] = batch
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    x = torch.randn(shape, generator=g, device=device, dtype=torch.float32)
    if name == "attn_softmax":
        return torch.softmax(x, dim=-1).contiguous()
    return torch.nn.functional.gelu(x).contiguous()


def config5_tensor_numpy(name: str, batch: int, seed: int = 0) -> np.ndarray:
    shape = list(CONFIG5_SHAPES[name])
    shape[0] = batch
    x = np.random.default_rng(seed).standard_normal(shape, dtype=np.float32)
    if name == "attn_softmax":
        e = np.exp(x - x.max(axis=-1, keepdims=True))
        return (e / e.sum(axis=-1, keepdims=True)).astype(np.float32)
    xd = x.astype(np.float64)
    erf = np.vectorize(math.erf)
    return (0.5 * xd * (1.0 + erf(xd / math.sqrt(2.0)))).astype(np.float32)


def dummy_layer_compute(a, b, reps: int) -> None:
    """Stand-in for a layer's kernels that run on the compute stream while a copy is in flight."""
    import torch

    for _ in range(reps):
        torch.mm(a, b)


def vgg16_modules(torch, dev):
    """VGG-16 feature extractor (conv/bn/relu x13, 5 pools; CSWAP+/vgg16-cifar10.cpp:77-97)."""
    mods = []
    cin = 3
    for c, reps in [(64, 2), (128, 2), (256, 3), (512, 3), (512, 3)]:
        for _ in range(reps):
            mods += [torch.nn.Conv2d(cin, c, 3, padding=1), torch.nn.BatchNorm2d(c), torch.nn.ReLU()]
            cin = c
        mods.append(torch.nn.MaxPool2d(2))
    return [m.to(dev) for m in mods]
