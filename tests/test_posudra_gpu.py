"""GPU numerics: the fp32-residual / score-modified attention kernels against
their plain-PyTorch fp32 references (dnet_amd.ops.reference), in bf16 and
fp32, at head sizes that are not powers of two, with ragged batches, slot
indirection and reused cache rows."""
import pytest
import torch

import dnet_amd.ops as ops
from dnet_amd.ops import reference as ref

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _tol(dt):
    return dict(atol=3e-2, rtol=3e-2) if dt == torch.bfloat16 \
        else dict(atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("dt_in,dt_out", [
    (torch.float32, torch.bfloat16), (torch.float32, torch.float32),
    (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("n", [40, 256, 1000, 4100])
def test_rmsnorm_rows(dt_in, dt_out, n):
    torch.manual_seed(n)
    x = (torch.randn(7, n, device=DEV) * 3).to(dt_in)
    w = torch.randn(n, device=DEV)
    y = ops.rmsnorm_rows(x, w, 1e-5, dt_out)
    yr = ref.rmsnorm_rows(x.cpu(), w.cpu(), 1e-5, dt_out)
    assert y.dtype == dt_out
    torch.testing.assert_close(y.cpu().float(), yr.float(), **_tol(dt_out))


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("two,norm", [(True, True), (False, True),
                                      (True, False)])
def test_ls_resid_rmsnorm(dt, two, norm):
    torch.manual_seed(3)
    n = 328
    h = torch.randn(5, n, device=DEV) * 4
    a = torch.randn(5, n, device=DEV).to(dt)
    b = torch.randn(5, n, device=DEV).to(dt) if two else None
    s1, s2 = torch.rand(n, device=DEV), torch.rand(n, device=DEV)
    wn = torch.randn(n, device=DEV) if norm else None
    hr = h.cpu().clone()
    yr = ref.ls_resid_rmsnorm(hr, a.cpu(), s1.cpu(),
                              b.cpu() if two else None,
                              s2.cpu() if two else None,
                              wn.cpu() if norm else None, 1e-5, dt)
    y = ops.ls_resid_rmsnorm(h, a, s1, b, s2 if two else None, wn, 1e-5, dt)
    torch.testing.assert_close(h.cpu(), hr, atol=1e-6, rtol=1e-6)
    if norm:
        torch.testing.assert_close(y.cpu().float(), yr.float(), **_tol(dt))
    else:
        assert y is None


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
def test_xielu(dt):
    torch.manual_seed(4)
    z = (torch.randn(9, 777, device=DEV) * 3).to(dt)
    for pq in ([0.3, -0.7], [-2.0, 1.5], [25.0, 0.0]):
        pq = torch.tensor(pq, device=DEV)
        y = ops.xielu(z, pq)
        yr = ref.xielu(z.cpu(), pq.cpu())
        torch.testing.assert_close(y.cpu().float(), yr.float(), **_tol(dt))


def _mods(hq, seed):
    g = torch.Generator().manual_seed(seed)
    return dict(temp=torch.rand(hq, generator=g) + 0.5,
                dist_r1=torch.rand(hq, generator=g),
                dist_r2=torch.rand(hq, generator=g) + 0.05,
                sinks=torch.randn(hq, generator=g))


CASES = [  # hq, hkv, d, dv, T, lens, pos0, slots, n_slots, smax
    (8, 4, 64, 48, 1, None, [5, 0, 130], None, 3, 200),          # decode
    (6, 2, 40, 24, 1, None, [63, 64, 65, 199], [3, 0, 5, 1], 6, 200),
    (4, 1, 128, 128, 37, [37, 1, 20], [0, 0, 0], [2, 0, 1], 3, 96),
    (3, 3, 20, 12, 70, [70, 33], [64, 127], [1, 0], 2, 256),     # continued
    (32, 1, 32, 16, 9, [9, 4], [0, 3], None, 2, 80),             # G > 16
    (2, 2, 256, 256, 3, None, [10], None, 1, 70),
    # decode against a long cache: the split-KV path and its combine
    (8, 2, 64, 64, 1, None, [5, 300, 511, 0], None, 4, 600),
    (6, 3, 40, 24, 1, None, [2000, 64, 1023], [2, 0, 1], 3, 2100),
    # prompts long enough for the matrix-core kernel (bf16), every tile class
    (8, 4, 64, 48, 200, [200, 77, 130], [0, 0, 0], [1, 2, 0], 3, 256),
    (4, 2, 192, 128, 70, [70, 3], [64, 10], None, 2, 160),
    (2, 1, 256, 256, 40, None, [0], None, 1, 64),
    (4, 4, 96, 72, 33, None, [31, 0], None, 2, 80),
    (2, 2, 16, 8, 129, [129, 64], [0, 1], None, 2, 200),
]


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("case", CASES)
def test_qknorm_append_and_attn_mod(dt, case):
    hq, hkv, d, dv, T, lens, pos0, slots, ns, smax = case
    torch.manual_seed(hq * 100 + d)
    B = len(pos0)
    kc = torch.randn(ns, hkv, smax, d).to(dt)
    vc = torch.randn(ns, hkv, smax, dv).to(dt)
    qkv = torch.randn(B * T, (hq + hkv) * d + hkv * dv).to(dt)
    qw, kw = torch.rand(hq * d) + 0.5, torch.rand(hkv * d) + 0.5
    pos = torch.tensor(pos0, dtype=torch.int32)
    lens_t = torch.tensor(lens, dtype=torch.int32) if lens else None
    slots_t = torch.tensor(slots, dtype=torch.int32) if slots else None
    mods = _mods(hq, d)
    for per_head in (False, True):
        qw_, kw_ = (qw[:d], kw[:d]) if per_head else (qw, kw)
        kr, vr = kc.clone(), vc.clone()
        qr = ref.qknorm_append(qkv, qw_, kw_, 1e-5, hq, hkv, d, dv, kr, vr,
                               pos, T, lens_t, slots_t, per_head)
        kg, vg = kc.to(DEV), vc.to(DEV)
        dev = lambda t: None if t is None else t.to(DEV)
        qg = ops.qknorm_append(qkv.to(DEV), qw_.to(DEV), kw_.to(DEV), 1e-5,
                               hq, hkv, d, dv, kg, vg, pos.to(DEV), T,
                               dev(lens_t), dev(slots_t), per_head)
        torch.testing.assert_close(kg.cpu().float(), kr.float(), **_tol(dt))
        assert torch.equal(vg.cpu(), vr)
        rows = [b * T + t for b in range(B)
                for t in range(lens[b] if lens else T)]
        torch.testing.assert_close(qg.cpu().float()[rows], qr.float()[rows],
                                   **_tol(dt))
        for window in (0, 17):
            kw_args = dict(softcap=2.5, window=window)
            ar = ref.attn_mod(qr, kr, vr, pos, T, 0.2, lens_t, slots_t,
                              **mods, **kw_args)
            ag = ops.attn_mod(qr.to(DEV), kr.to(DEV), vr.to(DEV),
                              pos.to(DEV), T, 0.2, dev(lens_t), dev(slots_t),
                              **{k: v.to(DEV) for k, v in mods.items()},
                              **kw_args)
            torch.testing.assert_close(ag.cpu().float()[rows],
                                       ar.float()[rows], **_tol(dt))
    # every modifier off: plain causal softmax attention
    ar = ref.attn_mod(qr, kr, vr, pos, T, 0.2, lens_t, slots_t)
    ag = ops.attn_mod(qr.to(DEV), kr.to(DEV), vr.to(DEV), pos.to(DEV), T, 0.2,
                      dev(lens_t), dev(slots_t))
    torch.testing.assert_close(ag.cpu().float()[rows], ar.float()[rows],
                               **_tol(dt))
