"""The committed fixtures (tests/golden/vectors.npz, written by tests/golden/make_vectors.py from
loop-level numpy statements of the operators) checked against the CPU oracle here and, on the
GPU box, against the HIP library through its C ABI.

Masks and the elementwise operators (sparsify, activation/truncation, add) must match bit for
bit; contractions and pooling within 1e-4 relative (fp32) / 2e-2 absolute (fp16).
"""
import os

import numpy as np
import pytest
import torch

from oracle import delta_ops as O
from util import DEV, cl, poison

V = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz"))
CONVS = sorted({k.split(".")[0] for k in V.files if k.endswith(".w") and not k.startswith("deconv")})
DECONVS = sorted({k.split(".")[0] for k in V.files if k.startswith("deconv") and k.endswith(".w")})
POOLS = sorted({k.split(".")[0] for k in V.files if k.endswith(".prev") and (k.startswith("max") or k.startswith("avg"))})
SPARSIFY = sorted({k.split(".")[0] for k in V.files if k.startswith("sparsify")})
ACTS = sorted({k.split(".")[0] for k in V.files if k.startswith("act")})
ADDS = sorted({k.split(".")[0] for k in V.files if k.startswith("add")})
DTYPES = [torch.float32, torch.float16]


def t(name):
    return torch.from_numpy(V[name])


def close(got, want, mask, dtype):
    m = (mask != 0).expand_as(want)
    g, w = got.float().cpu()[m], want.float()[m]
    if dtype == torch.float32:
        assert bool(((g - w).abs() <= 1e-5 + 1e-4 * w.abs()).all()), float((g - w).abs().max())
    else:
        assert bool(((g - w).abs() <= 2e-2).all()), float((g - w).abs().max())


def conv_cfg(name):
    c = [int(v) for v in V[f"{name}.cfg"]]
    return (c[0], c[1]), tuple(c[2:6]), (c[6], c[7]), c[8]


# ----------------------------------------------------------------------------- CPU: the oracle
@pytest.mark.parametrize("name", CONVS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_oracle_conv(name, dtype):
    s, p, d, g = conv_cfg(name)
    out, om = O.conv(t(f"{name}.x").to(dtype), t(f"{name}.mask"), t(f"{name}.w").to(dtype),
                     t(f"{name}.b").to(dtype), s, p, d, g)
    assert torch.equal(om, t(f"{name}.out_mask"))
    close(out, t(f"{name}.out"), om, dtype)


@pytest.mark.parametrize("name", DECONVS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_oracle_deconv(name, dtype):
    s, p = (int(v) for v in V[f"{name}.cfg"])
    out, om = O.deconv(t(f"{name}.x").to(dtype), t(f"{name}.mask"), t(f"{name}.w").to(dtype),
                       t(f"{name}.b").to(dtype), (s, s), (p, p))
    assert torch.equal(om, t(f"{name}.out_mask"))
    close(out, t(f"{name}.out"), om, dtype)


def pool_cfg(name):
    c = [int(v) for v in V[f"{name}.cfg"]]
    return (c[0], c[1]), (c[2], c[3]), tuple(c[4:8]), c[8]


@pytest.mark.parametrize("name", POOLS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_oracle_pool(name, dtype):
    k, s, p, mode = pool_cfg(name)
    out, om = O.pool(t(f"{name}.x").to(dtype), t(f"{name}.prev").to(dtype), t(f"{name}.mask"), k, s, p, (1, 1), mode)
    assert torch.equal(om, t(f"{name}.out_mask"))
    close(out, t(f"{name}.out"), om, dtype)


@pytest.mark.parametrize("name", SPARSIFY)
def test_oracle_sparsify(name):
    prev = t(f"{name}.prev").clone()
    delta, mask = O.sparsify(t(f"{name}.x"), prev, 0.1)
    assert torch.equal(mask, t(f"{name}.mask")) and torch.equal(delta, t(f"{name}.delta"))
    assert torch.equal(prev, t(f"{name}.new_prev"))


@pytest.mark.parametrize("name", ACTS)
def test_oracle_activate_truncate(name):
    act = int(name[3])
    a = [t(f"{name}.{k}").clone() for k in ("delta", "prev", "trunc", "mask")]
    O.activate_truncate(*a, 0.05, act, O.TRUNC_MAX)
    assert torch.equal(a[3], t(f"{name}.out_mask"))
    assert torch.equal(a[1], t(f"{name}.out_prev")) and torch.equal(a[2], t(f"{name}.out_trunc"))
    m = (a[3] != 0).expand_as(a[0])
    assert torch.equal(a[0][m], t(f"{name}.out_delta")[m])


@pytest.mark.parametrize("name", ADDS)
def test_oracle_add(name):
    out, mo = O.add(t(f"{name}.a"), t(f"{name}.mask_a"), t(f"{name}.b"), t(f"{name}.mask_b"), None, 0.75, 1.5)
    assert torch.equal(mo, t(f"{name}.out_mask")) and torch.equal(out, t(f"{name}.out"))


# ------------------------------------------------------------------- GPU: the HIP library (C ABI)
def hk():
    import deltacnn_amd.hip_kernels as m
    return m


def _filter(w, dtype, depthwise, transposed=False):
    from deltacnn_amd.filter_conversion import convert_filter_out_channels_last, convert_half_filter
    if dtype == torch.float16:
        return convert_half_filter(w, pixel_wise=depthwise, transposed=transposed)
    return convert_filter_out_channels_last(w, transposed=transposed)


@pytest.mark.gpu
@pytest.mark.parametrize("name", CONVS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_conv(lib, name, dtype):
    s, p, d, g = conv_cfg(name)
    x, mask, w = t(f"{name}.x").to(dtype), t(f"{name}.mask"), t(f"{name}.w").to(dtype)
    filt = _filter(w, dtype, g > 1).to(DEV)
    out, om = hk().sparse_conv(cl(poison(x, mask)), filt, cl(mask), t(f"{name}.b").to(dtype).to(DEV), s, p, d, g,
                               c_out=w.shape[0], create_out_mask=True)
    assert torch.equal(om.cpu(), t(f"{name}.out_mask"))
    close(out, t(f"{name}.out"), om.cpu(), dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("name", DECONVS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_deconv(lib, name, dtype):
    s, p = (int(v) for v in V[f"{name}.cfg"])
    x, mask, w = t(f"{name}.x").to(dtype), t(f"{name}.mask"), t(f"{name}.w").to(dtype)
    filt = _filter(w, dtype, False, True).to(DEV)
    out, om = hk().sparse_deconv(cl(poison(x, mask)), filt, cl(mask), t(f"{name}.b").to(dtype).to(DEV), (s, s),
                                 (p, p), (1, 1), 1, c_out=w.shape[1], create_out_mask=True)
    assert torch.equal(om.cpu(), t(f"{name}.out_mask"))
    close(out, t(f"{name}.out"), om.cpu(), dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("name", POOLS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_pool(lib, name, dtype):
    k, s, p, mode = pool_cfg(name)
    x, mask = t(f"{name}.x").to(dtype), t(f"{name}.mask")
    out, om = hk().sparse_pooling(cl(poison(x, mask)), cl(t(f"{name}.prev").to(dtype)), k, cl(mask), s, p,
                                  pooling_mode_int=mode)
    assert torch.equal(om.cpu(), t(f"{name}.out_mask"))
    close(out, t(f"{name}.out"), om.cpu(), dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("name", SPARSIFY)
def test_hip_sparsify(lib, name):
    x, prev = cl(t(f"{name}.x")), cl(t(f"{name}.prev"))
    delta = torch.full_like(x, float("nan"))
    mask = torch.full((x.shape[0], 1, x.shape[2], x.shape[3]), -3, dtype=torch.int32, device=DEV)
    hk().sparsify(x, prev, delta, mask, 0.1)
    want_mask = t(f"{name}.mask")
    assert torch.equal(mask.cpu(), want_mask) and torch.equal(prev.cpu(), t(f"{name}.new_prev"))
    m = (want_mask != 0).expand_as(delta)
    assert torch.equal(delta.cpu()[m], t(f"{name}.delta")[m])


@pytest.mark.gpu
@pytest.mark.parametrize("name", ACTS)
def test_hip_activate_truncate(lib, name):
    act = int(name[3])
    delta, mask = t(f"{name}.delta"), t(f"{name}.mask")
    a = [cl(poison(delta, mask)), cl(t(f"{name}.prev")), cl(t(f"{name}.trunc")), cl(mask)]
    hk().sparse_activation(*a, 0.05, act, 0)
    assert torch.equal(a[3].cpu(), t(f"{name}.out_mask"))
    assert torch.equal(a[1].cpu(), t(f"{name}.out_prev")) and torch.equal(a[2].cpu(), t(f"{name}.out_trunc"))
    m = (t(f"{name}.out_mask") != 0).expand_as(delta)
    assert torch.equal(a[0].cpu()[m], t(f"{name}.out_delta")[m])


@pytest.mark.gpu
@pytest.mark.parametrize("name", ADDS)
def test_hip_add(lib, name):
    a, b, ma, mb = t(f"{name}.a"), t(f"{name}.b"), t(f"{name}.mask_a"), t(f"{name}.mask_b")
    da, db = cl(poison(a, ma)), cl(poison(b, mb))
    out = torch.full_like(da, float("nan"))
    mo = torch.full_like(cl(ma), -3)
    hk().sparse_add_tensors(da, db, None, out, cl(ma), cl(mb), mo, 0.75, 1.5, 0, False)
    want_mask = t(f"{name}.out_mask")
    assert torch.equal(mo.cpu(), want_mask)
    m = (want_mask != 0).expand_as(a)
    assert torch.equal(out.cpu()[m], t(f"{name}.out")[m])
