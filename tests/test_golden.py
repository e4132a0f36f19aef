"""The committed golden vectors (``tests/golden/*.npz``, written by ``tests/golden/make_golden.py`` from
PyTorch's math SDPA under forward-mode AD in fp64) against the CPU restatements in ``oracle/`` and,
on a GPU, against the HIP kernels through the C ABI."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import dense, tiled

HERE = os.path.dirname(os.path.abspath(__file__))
FILES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))
NAMES = [os.path.splitext(os.path.basename(f))[0] for f in FILES]
INPUTS = ("q", "k", "v", "qt", "kt", "vt", "go", "gt")
GRADS = ("dq", "dk", "dv", "dqt", "dkt", "dvt")


def _load(path):
    with np.load(path, allow_pickle=False) as z:
        return {n: z[n] for n in z.files}


def test_the_fixtures_are_there():
    assert len(FILES) == 6


@pytest.mark.parametrize("path", FILES, ids=NAMES)
def test_dense_oracle_reproduces_the_golden_vectors(path):
    c = _load(path)
    x = [c[n].astype(np.float64) for n in INPUTS]
    mask = c.get("mask")
    if mask is not None and mask.dtype != np.bool_:
        mask = mask.astype(np.float64)
    fw = dense.forward(*x[:6], mask=mask, causal=bool(c["causal"]), scale=float(c["scale"]))
    bw = dense.backward(*x, mask=mask, causal=bool(c["causal"]), scale=float(c["scale"]))
    for n in ("O", "Ot", "M", "mu"):
        np.testing.assert_allclose(fw[n], c[n], rtol=2e-6, atol=2e-6, err_msg=n)
    for n in GRADS:
        np.testing.assert_allclose(bw[n], c[n], rtol=2e-6, atol=2e-6, err_msg=n)


@pytest.mark.parametrize("path", FILES, ids=NAMES)
def test_tiled_oracle_reproduces_the_golden_vectors(path):
    c = _load(path)
    x = [torch.from_numpy(c[n]).double() for n in INPUTS]
    mask = c.get("mask")
    if mask is not None:
        mask = torch.from_numpy(mask)
        mask = mask if mask.dtype == torch.bool else mask.double()
    kw = dict(mask=mask, causal=bool(c["causal"]), scale=float(c["scale"]), bm=32, bn=32)
    o, ot, M, mu = tiled.forward(*x[:6], **kw)
    grads = tiled.backward(*x[:6], o, ot, M, mu, x[6], x[7], **kw)
    for n, t in zip(("O", "Ot", "M", "mu") + GRADS, (o, ot, M, mu, *(grads[g] for g in GRADS))):
        np.testing.assert_allclose(t.numpy(), c[n], rtol=2e-6, atol=2e-6, err_msg=n)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("path", FILES, ids=NAMES)
def test_hip_kernels_reproduce_the_golden_vectors(path, dt):
    """fp32: max-abs <= 1e-4; bf16 / fp16: max|x - ref| / max|ref| <= 2e-2.  The inputs are
    bf16-representable, so every element type computes on exactly the stored numbers."""
    from jvp_flash_attention_amd import _lib

    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[dt]
    c = _load(path)
    dev = [torch.from_numpy(c[n]).to(dtype).cuda() for n in INPUTS]
    mask, kind = None, _lib.MASK_NONE
    if "mask" in c:
        m = torch.from_numpy(c["mask"])
        mask, kind = (m.cuda(), _lib.MASK_BOOL) if m.dtype == torch.bool else (m.to(dtype).cuda(), _lib.MASK_ADD)
    causal, scale = bool(c["causal"]), float(c["scale"])
    print(f"case golden {os.path.basename(path)} {dt}", flush=True)
    be = _lib.backend()
    o, ot, M, mu = be.fwd(*dev[:6], mask, kind, causal, scale)
    grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], mask, kind, causal, scale, want_tangent_grads=True)
    got = dict(zip(("O", "Ot", "M", "mu") + GRADS, (o, ot, M, mu, *grads)))
    for n, t in got.items():
        t = t.double().cpu().numpy()
        assert np.isfinite(t).all(), n
        err = np.abs(t - c[n]).max()
        if dtype == torch.float32:
            assert err <= 1e-4, f"{n}: max-abs {err:.3e}"
        else:
            assert err / np.abs(c[n]).max() <= 2e-2, f"{n}: relative {err / np.abs(c[n]).max():.3e}"
