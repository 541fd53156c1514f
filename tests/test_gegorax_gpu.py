"""GPU numerics: the sequence-state kernels (pooled-block attention, rotation
in the q/k-norm append, causal convolution, the two recurrences, grouped gated
norm, branch-sum residual update and the small element-wise steps) against
their plain-PyTorch fp32 references (dnet_amd.ops.reference), in bf16 and
fp32, with ragged batches, slot indirection, continued states and sizes that
are not multiples of the kernels' tiles."""
import pytest
import torch

import dnet_amd.ops as ops
from dnet_amd.ops import reference as ref

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTS = [torch.bfloat16, torch.float32]


def _tol(dt):
    return dict(atol=3e-2, rtol=3e-2) if dt == torch.bfloat16 \
        else dict(atol=3e-5, rtol=3e-5)


def _geo(B, T, lens, slots, pos):
    i32 = lambda v: torch.tensor(v, dtype=torch.int32)
    return i32(pos), i32(lens), i32(slots)


def _both(fn, *tensors):
    """Run fn on CPU copies (reference) and on the GPU tensors."""
    return fn([t.cpu() if torch.is_tensor(t) else t for t in tensors])


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("d,nrot", [(32, 16), (24, 5), (7, 3), (96, 48)])
def test_qknorm_rotation_append(dt, d, nrot):
    torch.manual_seed(d)
    nq, nkv, dv, T, B, Bc, S = 4, 2, 12, 5, 3, 4, 64
    qkv = torch.randn(B * T, (nq + nkv) * d + nkv * dv, device=DEV).to(dt)
    qw, kw = torch.randn(d, device=DEV), torch.randn(d, device=DEV)
    freq = (10000.0 ** (-torch.arange(nrot) / nrot)).float().to(DEV)
    pos, lens, slots = _geo(B, T, [5, 2, 0], [3, 0, 1], [40, 0, 7])
    kc = torch.zeros(Bc, nkv, S, d, device=DEV, dtype=dt)
    vc = torch.zeros(Bc, nkv, S, dv, device=DEV, dtype=dt)
    kr, vr = kc.cpu().clone(), vc.cpu().clone()
    q = ops.qknorm_append(qkv, qw, kw, 1e-5, nq, nkv, d, dv, kc, vc,
                          pos.to(DEV), T, lens.to(DEV), slots.to(DEV),
                          per_head=True, rot_freq=freq)
    qr = ref.qknorm_append(qkv.cpu(), qw.cpu(), kw.cpu(), 1e-5, nq, nkv, d,
                           dv, kr, vr, pos, T, lens, slots, True, freq.cpu())
    torch.testing.assert_close(q.cpu().float(), qr.float(), **_tol(dt))
    torch.testing.assert_close(kc.cpu().float(), kr.float(), **_tol(dt))
    torch.testing.assert_close(vc.cpu().float(), vr.float(), **_tol(dt))


def _pool_case(dt, T, pos, lens, slots, Hq=4, Hkv=2, D=32, DV=16, window=20,
               pool=4, S=256, Bc=4, seed=0):
    torch.manual_seed(seed)
    B = len(pos)
    kc = torch.randn(Bc, Hkv, S, D, device=DEV).to(dt)
    vc = torch.randn(Bc, Hkv, S, DV, device=DEV).to(dt)
    Sp = S // pool + 1
    pk = torch.zeros(Bc, Hkv, Sp, D, device=DEV, dtype=dt)
    pv = torch.zeros(Bc, Hkv, Sp, DV, device=DEV, dtype=dt)
    # pooled entries of everything before this step: one call from 0
    z = torch.zeros(B, dtype=torch.int32)
    p, l, s = _geo(B, T, lens, slots, pos)
    full = (p + l).clamp(min=1)
    Tm = int(full.max())
    pkr, pvr = pk.cpu().clone(), pv.cpu().clone()
    ops.kv_pool_update(kc, vc, pk, pv, z.to(DEV), Tm, pool, full.to(DEV),
                       s.to(DEV))
    ref.kv_pool_update(kc.cpu(), vc.cpu(), pkr, pvr, z, Tm, pool, full, s)
    torch.testing.assert_close(pk.cpu().float(), pkr.float(), **_tol(dt))
    torch.testing.assert_close(pv.cpu().float(), pvr.float(), **_tol(dt))
    q = torch.randn(B * T, Hq * D, device=DEV).to(dt)
    out = ops.attn_mod(q, kc, vc, p.to(DEV), T, 0.2, l.to(DEV), s.to(DEV),
                       window=window, pool_k=pk, pool_v=pv, pool=pool)
    want = ref.attn_mod(q.cpu(), kc.cpu(), vc.cpu(), p, T, 0.2, l, s,
                        window=window, pool_k=pkr, pool_v=pvr, pool=pool)
    torch.testing.assert_close(out.cpu().float(), want.float(), **_tol(dt))


@pytest.mark.parametrize("dt", DTS)
def test_pooled_window_attention_decode(dt):
    _pool_case(dt, 1, [200, 19, 20, 0], [1, 1, 1, 0], [2, 0, 3, 1])
    _pool_case(dt, 1, [130, 23], [1, 1], [1, 0], Hq=6, Hkv=2, D=24, DV=40,
               window=17, pool=3, seed=1)


@pytest.mark.parametrize("dt", DTS)
def test_pooled_window_attention_prompt(dt):
    _pool_case(dt, 70, [0, 100, 33], [70, 41, 3], [3, 1, 0])
    _pool_case(dt, 40, [90, 0], [40, 17], [0, 2], Hq=2, Hkv=1, D=64, DV=64,
               window=32, pool=8, seed=2)
    _pool_case(dt, 18, [60], [18], [1], Hq=3, Hkv=3, D=20, DV=12, window=9,
               pool=5, seed=3)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("taps", [4, 2, 1])
def test_causal_conv_silu(dt, taps):
    torch.manual_seed(taps)
    C, T, B, Bc, col0, ld = 70, 6, 3, 4, 9, 100
    x = torch.randn(B * T, ld, device=DEV).to(dt)
    w, b = torch.randn(C, taps, device=DEV), torch.randn(C, device=DEV)
    st = torch.randn(Bc, taps - 1, C, device=DEV).to(dt)
    str_ = st.cpu().clone()
    pos, lens, slots = _geo(B, T, [6, 1, 0], [2, 0, 3], [0, 1, 9])
    for _ in range(2):          # the second call continues the first
        y = ops.causal_conv_silu(x, col0, w, b, st, pos.to(DEV), T,
                                 lens.to(DEV), slots.to(DEV))
        yr = ref.causal_conv_silu(x.cpu(), col0, w.cpu(), b.cpu(), str_, pos,
                                  T, lens, slots)
        torch.testing.assert_close(y.cpu(), yr, atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(st.cpu().float(), str_.float())
        pos = pos + lens


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("heads,P,N,G", [(4, 32, 32, 2), (3, 20, 40, 1),
                                         (8, 64, 128, 2), (2, 8, 16, 2)])
def test_ssd_scan(dt, heads, P, N, G):
    torch.manual_seed(N)
    T, B, Bc = 37, 3, 4
    inner = heads * P
    xbc = torch.randn(B * T, inner + 2 * G * N, device=DEV) * 0.5
    dts = torch.randn(B * T, heads + 5, device=DEV).to(dt)
    dtb = torch.randn(heads, device=DEV) - 1
    al, dk = torch.rand(heads, device=DEV), torch.randn(heads, device=DEV)
    st = torch.randn(Bc, heads, N, P, device=DEV)
    str_ = st.cpu().clone()
    pos, lens, slots = _geo(B, T, [37, 5, 0], [1, 3, 0], [0, 12, 4])
    for _ in range(2):
        y = ops.ssd_scan(xbc, dts, 3, dtb, al, dk, st, pos.to(DEV), T, heads,
                         P, N, G, lens.to(DEV), slots.to(DEV))
        yr = ref.ssd_scan(xbc.cpu(), dts.cpu(), 3, dtb.cpu(), al.cpu(),
                          dk.cpu(), str_, pos, T, heads, P, N, G, lens, slots)
        n0 = int(lens[0])
        torch.testing.assert_close(y.cpu()[:n0], yr[:n0], atol=2e-4,
                                   rtol=2e-4)
        torch.testing.assert_close(y.cpu()[T:T + 5], yr[T:T + 5], atol=2e-4,
                                   rtol=2e-4)
        torch.testing.assert_close(st.cpu(), str_, atol=2e-4, rtol=2e-4)
        pos = pos + lens


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,d", [(2, 64), (3, 24), (1, 128), (2, 8)])
def test_delta_scan(dt, H, d):
    torch.manual_seed(d)
    T, B, Bc = 29, 3, 4
    n = H * d
    src = torch.randn(B * T, 5 * n + 6, device=DEV).to(dt)
    wl = torch.randn(B * T, n, device=DEV).to(dt)
    w0, ab = torch.randn(n, device=DEV), torch.randn(n, device=DEV)
    st = torch.randn(Bc, H, d, d, device=DEV) * 0.3
    str_ = st.cpu().clone()
    pos, lens, slots = _geo(B, T, [29, 4, 0], [3, 1, 0], [0, 6, 2])
    for _ in range(2):
        o = ops.delta_scan(src, 0, n, 2 * n, 4 * n, wl, w0, ab, st,
                           pos.to(DEV), T, H, d, 0.6, 1e-6, lens.to(DEV),
                           slots.to(DEV))
        orf = ref.delta_scan(src.cpu(), 0, n, 2 * n, 4 * n, wl.cpu(),
                             w0.cpu(), ab.cpu(), str_, pos, T, H, d, 0.6,
                             1e-6, lens, slots)
        for lo, hi in ((0, int(lens[0])), (T, T + 4)):
            torch.testing.assert_close(o.cpu()[lo:hi], orf[lo:hi], atol=3e-4,
                                       rtol=3e-4)
        torch.testing.assert_close(st.cpu(), str_, atol=3e-4, rtol=3e-4)
        pos = pos + lens


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("silu,first,groups,N", [(True, True, 2, 128),
                                                 (False, False, 3, 60),
                                                 (True, False, 1, 200),
                                                 (False, True, 8, 64),
                                                 (True, True, 1, 2048),
                                                 (False, False, 2, 2050)])
def test_gated_group_rmsnorm(dt, silu, first, groups, N):
    torch.manual_seed(N)
    M = 9
    y = torch.randn(M, N, device=DEV)
    gs = torch.randn(M, N + 11, device=DEV).to(dt)
    w = torch.randn(N, device=DEV)
    kind = "silu" if silu else "sigmoid"
    out = ops.gated_group_rmsnorm(y, gs, 7, w, groups, 1e-5, kind, first, dt)
    want = ref.gated_group_rmsnorm(y.cpu(), gs.cpu(), 7, w.cpu(), groups,
                                   1e-5, kind, first, dt)
    torch.testing.assert_close(out.cpu().float(), want.float(), **_tol(dt))


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("N", [96, 130])
@pytest.mark.parametrize("mode", ["two_normed", "one_plain", "normed_next"])
def test_resid_branches_rmsnorm(dt, N, mode):
    torch.manual_seed(N)
    M = 6
    h = torch.randn(M, N, device=DEV) * 3
    a = torch.randn(M, N, device=DEV).to(dt)
    b = torch.randn(M, N, device=DEV).to(dt)
    f32 = torch.randn(M, N, device=DEV)
    wa, wb, wn = (torch.randn(N, device=DEV) for _ in range(3))
    if mode == "two_normed":
        args = (a, wa, b, wb, 0.5, f32, None)
        cast = True
    elif mode == "one_plain":
        args = (a, None, None, None, 1.0, f32.to(dt), wn)
        cast = False
    else:
        args = (a, wa, None, None, 1.0, None, wn)
        cast = True
    hr = h.cpu().clone()
    y, xc = ops.resid_branches_rmsnorm(h, *args, 1e-5, dt, cast)
    yr, xr = ref.resid_branches_rmsnorm(
        hr, *[t.cpu() if torch.is_tensor(t) else t for t in args], 1e-5, dt,
        cast)
    torch.testing.assert_close(h.cpu(), hr, atol=2e-5, rtol=2e-5)
    for got, want in ((y, yr), (xc, xr)):
        assert (got is None) == (want is None)
        if got is not None:
            torch.testing.assert_close(got.cpu().float(), want.float(),
                                       **_tol(dt))


@pytest.mark.parametrize("dt", DTS)
def test_small_elementwise_steps(dt):
    torch.manual_seed(5)
    x = (torch.randn(11, 50, device=DEV) * 2).to(dt)
    for kind in ("relu_sq", "tanh"):
        torch.testing.assert_close(
            ops.act_slice(x, 6, 33, kind).cpu().float(),
            ref.act_slice(x.cpu(), 6, 33, kind).float(), **_tol(dt))
    table = torch.randn(40, 90, device=DEV).to(dt)
    tok = torch.randint(0, 40, (11,), device=DEV)
    z = x[:, :24].contiguous()
    torch.testing.assert_close(
        ops.gelu_gather_mul(z, table, tok, 48).cpu().float(),
        ref.gelu_gather_mul(z.cpu(), table.cpu(), tok.cpu(), 48).float(),
        **_tol(dt))
    torch.testing.assert_close(
        ops.clamped_glu(x, 1.702, 1.5).cpu().float(),
        ref.clamped_glu(x.cpu(), 1.702, 1.5).float(), **_tol(dt))
