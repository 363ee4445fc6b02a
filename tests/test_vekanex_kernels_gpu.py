"""Each kernel call of the Vekanex mixers and of the routed experts alone, against the plain torch
function of the same name (tests/emulated_ops.py), in both activation types: steps of several
sequences of unequal length, some at their start in slots that hold another request's leftovers
(NaN here), some continuing; sizes that are no multiples of anything."""
import types

import pytest
import torch

from emulated_ops import EmulatedOps
from servelab_amd.kernels import HipOps

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def tables(dtype):
    return HipOps(dtype, DEV), EmulatedOps(dtype)


def fake_batch(q_lens, starts, slots, device):
    cu, pos, seq = [0], [], []
    for i, (n, s) in enumerate(zip(q_lens, starts)):
        cu.append(cu[-1] + n)
        pos += list(range(s, s + n))
        seq += [i] * n
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    return types.SimpleNamespace(cu_q=i32(cu), positions=i32(pos), tok_seq=i32(seq), state_slots=i32(slots),
                                 ctx_len=i32([s + n for n, s in zip(q_lens, starts)]),
                                 num_seqs=len(q_lens), num_tokens=cu[-1], q_lens=q_lens, starts=starts)


Q_LENS, STARTS, SLOTS = [1, 37, 2, 19, 1], [0, 5, 0, 7, 300], [4, 0, 5, 2, 1]


def states(n, width, seed):
    """Slots of random state; those of sequences at their start hold NaN, which must not be read."""
    g = torch.Generator().manual_seed(seed)
    st = torch.randn(n, width, generator=g) * 0.3
    for s, start in zip(SLOTS, STARTS):
        if start == 0:
            st[s] = float("nan")
    return st


def close(a, b, tol):
    a, b = a.float().cpu(), b.float().cpu()
    assert torch.isfinite(a).all()
    assert (a - b).abs().max() <= tol * max(1.0, float(b.abs().max())), float((a - b).abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
def test_postnorm_scaled_sum_softcap(dtype):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(0)
    for T, H in ((1, 72), (33, 256), (5, 2048 + 8)):
        resid = torch.randn(T, H, generator=g)
        y = torch.randn(T, H, generator=g).to(dtype)
        w = 1 + 0.3 * torch.randn(H, generator=g)
        r1, r2 = resid.clone().to(DEV), resid.clone()
        o1 = hip.add_postnorm(r1, y.to(DEV), w.to(DEV), 1e-5, 0.6)
        o2 = emu.add_postnorm(r2, y, w, 1e-5, 0.6)
        close(r1, r2, 1e-6)
        close(o1, o2, 1e-6 if dtype == torch.float32 else 8e-3)
        close(hip.add_postnorm(r1, None, w.to(DEV), 1e-5, 0.6), r1.cpu().to(dtype), 0)
        a, b = y, torch.randn(T, H, generator=g).to(dtype)
        close(hip.scaled_sum(a.to(DEV), 0.8, b.to(DEV), -1.3), emu.scaled_sum(a, 0.8, b, -1.3),
              1e-6 if dtype == torch.float32 else 8e-3)
        z = 40 * torch.randn(T, H, generator=g)
        close(hip.softcap(z.clone().to(DEV), 30.0), emu.softcap(z.clone(), 30.0), 1e-6)


def test_lowrank_expand_modes():
    hip, emu = tables(torch.float32)
    g = torch.Generator().manual_seed(1)
    T, heads = 23, 3
    for rank, per in ((4, 8), (24, 40), (16, 136)):
        C = heads * per
        buf = torch.randn(T, 50 + rank, generator=g)
        w2, bias, rates = torch.randn(C, rank, generator=g), torch.randn(C, generator=g), torch.randn(heads, generator=g)
        for mode, kw in (("plain", {}), ("log_sigmoid", {"divisor": 7.0}), ("rate_softplus", {"rates": rates})):
            dev = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in kw.items()}
            for b in (bias, None):
                got = hip.lowrank_expand(buf.to(DEV), 50, w2.to(DEV), None if b is None else b.to(DEV), mode,
                                         heads=heads, **dev)
                close(got, emu.lowrank_expand(buf, 50, w2, b, mode, heads=heads, **kw), 2e-6)


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_short_conv_keeps_its_last_inputs(taps):
    hip, emu = tables(torch.float32)
    g = torch.Generator().manual_seed(2)
    heads, dim, rest = 5, 24, 300
    C = heads * dim + rest
    T = sum(Q_LENS)
    buf = torch.randn(T, 7 + C, generator=g)
    w = torch.randn(C, taps, generator=g)
    off = 11
    st = states(6, off + (taps - 1) * C + 3, seed=3)
    batch_d, batch_h = fake_batch(Q_LENS, STARTS, SLOTS, DEV), fake_batch(Q_LENS, STARTS, SLOTS, "cpu")
    kw = dict(unit_heads=heads, unit_dim=dim, unit_eps=1e-6, scaled_heads=2, scale=dim ** -0.5)
    s1, s2 = st.clone().to(DEV), st.clone()
    o1 = hip.short_conv(buf.to(DEV), 7, w.to(DEV), s1, off, batch_d, True, **kw)
    o2 = emu.short_conv(buf, 7, w, s2, off, batch_h, True, **kw)
    close(o1, o2, 2e-6)
    used = sorted(SLOTS)
    if taps > 1:
        close(s1[used][:, off:off + (taps - 1) * C], s2[used][:, off:off + (taps - 1) * C], 0)
    assert torch.equal(torch.nan_to_num(s1.cpu()[:, :off], 9.0), torch.nan_to_num(st[:, :off], 9.0))
    s3 = st.clone().to(DEV)
    hip.short_conv(buf.to(DEV), 7, w.to(DEV), s3, off, batch_d, False, **kw)          # a reading call leaves the slot
    assert torch.equal(torch.nan_to_num(s3.cpu(), 9.0), torch.nan_to_num(st, 9.0))


@pytest.mark.parametrize("H,G,D,Dv", [(2, 2, 8, 16), (4, 2, 24, 8), (4, 1, 72, 32), (1, 1, 136, 70), (3, 3, 40, 300)])
@pytest.mark.parametrize("delta", [False, True])
def test_decay_scan(H, G, D, Dv, delta):
    hip, emu = tables(torch.float32)
    g = torch.Generator().manual_seed(4)
    T = sum(Q_LENS)
    width = 3 + 2 * G * D + H * Dv
    src = torch.randn(T, width, generator=g) * 0.5
    log_decay = -torch.rand(T, H * D, generator=g) * 0.3
    beta = torch.randn(T, 5 + H, generator=g) if delta else None
    st = states(6, H * D * Dv + 9, seed=5)
    bd, bh = fake_batch(Q_LENS, STARTS, SLOTS, DEV), fake_batch(Q_LENS, STARTS, SLOTS, "cpu")
    s1, s2 = st.clone().to(DEV), st.clone()
    args = (3, 3 + G * D, 3 + 2 * G * D, H, G, D, Dv)
    o1 = hip.decay_scan(src.to(DEV), *args, log_decay.to(DEV), 0.7, None if beta is None else beta.to(DEV), 5, s1, bd, True)
    o2 = emu.decay_scan(src, *args, log_decay, 0.7, beta, 5, s2, bh, True)
    close(o1, o2, 1e-5)
    used = sorted(SLOTS)
    close(s1[used][:, :H * D * Dv], s2[used][:, :H * D * Dv], 1e-5)
    assert torch.equal(torch.nan_to_num(s1.cpu()[:, H * D * Dv:], 9.0), torch.nan_to_num(st[:, H * D * Dv:], 9.0))


@pytest.mark.parametrize("H,D,Dv", [(2, 8, 16), (3, 24, 8), (1, 72, 40), (2, 136, 16)])
def test_mlstm_scan(H, D, Dv):
    hip, emu = tables(torch.float32)
    g = torch.Generator().manual_seed(6)
    T = sum(Q_LENS)
    width = 2 * H * D + H * Dv + 2 * H + 1
    buf = torch.randn(T, width, generator=g)
    buf[:, -2 * H - 1:] *= 6.0                                       # gates beyond their cap as well
    n = H * D * Dv + H * D + H
    st = states(6, n, seed=7)
    st[:, -H:] = st[:, -H:].abs() * 5                                # running maxima
    bd, bh = fake_batch(Q_LENS, STARTS, SLOTS, DEV), fake_batch(Q_LENS, STARTS, SLOTS, "cpu")
    s1, s2 = st.clone().to(DEV), st.clone()
    cols = (0, H * D, 2 * H * D, 2 * H * D + H * Dv, 2 * H * D + H * Dv + H)
    o1 = hip.mlstm_scan(buf.to(DEV), *cols, H, D, Dv, 4.0, D ** -0.5, s1, bd, True)
    o2 = emu.mlstm_scan(buf, *cols, H, D, Dv, 4.0, D ** -0.5, s2, bh, True)
    close(o1, o2, 2e-5)
    close(s1[sorted(SLOTS)], s2[sorted(SLOTS)], 2e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_head_norm_gate(dtype):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(8)
    for H, Dv in ((2, 16), (3, 70), (1, 300)):
        o = torch.randn(9, H * Dv, generator=g)
        gate = torch.randn(9, 4 + H * Dv, generator=g)
        for per_head, act in ((True, "sigmoid"), (False, "silu")):
            w = 1 + 0.2 * torch.randn(H * Dv if per_head else Dv, generator=g)
            close(hip.head_norm_gate(o.to(DEV), H, Dv, w.to(DEV), per_head, 1e-5, gate.to(DEV), 4, act),
                  emu.head_norm_gate(o, H, Dv, w, per_head, 1e-5, gate, 4, act),
                  2e-6 if dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,rot", [(4, 2, 16, 24, 8), (3, 1, 8, 8, 8), (8, 1, 96, 64, 24), (2, 2, 40, 16, 0)])
def test_projnorm_rope_store(dtype, H, G, D, Dv, rot):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(9)
    T, page, pages = 21, 16, 5
    buf = torch.randn(T, (H + G) * D + G * Dv + 3, generator=g)
    qg, kg = 1 + 0.2 * torch.randn(H * D, generator=g), 1 + 0.2 * torch.randn(G * D, generator=g)
    pos = torch.randint(0, 900, (T,), generator=g)
    inv = 1.0 / (500.0 ** (torch.arange(0, max(rot, 2), 2).float() / max(rot, 2)))
    ang = pos.float()[:, None] * inv[None, :]
    tab = types.SimpleNamespace(cos=torch.cos(ang), sin=torch.sin(ang))
    tab_d = types.SimpleNamespace(cos=tab.cos.to(DEV), sin=tab.sin.to(DEV))
    slots = torch.randperm(page * pages, generator=g)[:T].to(torch.int32)
    k1 = torch.full((pages, G, page, D), float("nan"), dtype=dtype)
    v1 = torch.full((pages, G, Dv, page), float("nan"), dtype=dtype)
    k2, v2 = k1.clone(), v1.clone()
    k1, v1 = k1.to(DEV), v1.to(DEV)
    q1 = hip.projnorm_rope_store(buf.to(DEV), H, G, D, Dv, qg.to(DEV), kg.to(DEV), 1e-5, rot, tab_d if rot else None,
                                 slots.to(DEV), k1, v1, page)
    q2 = emu.projnorm_rope_store(buf, H, G, D, Dv, qg, kg, 1e-5, rot, tab if rot else None, slots, k2, v2, page)
    tol = 3e-6 if dtype == torch.float32 else 8e-3
    close(q1, q2, tol)
    written = ~torch.isnan(k2.float())
    assert torch.equal(~torch.isnan(k1.float().cpu()), written)
    close(torch.nan_to_num(k1.float()), torch.nan_to_num(k2.float()), tol)
    close(torch.nan_to_num(v1.float()), torch.nan_to_num(v2.float()), tol)


@pytest.mark.parametrize("T,E,top", [(1, 5, 2), (7, 12, 4), (200, 64, 8), (33, 3, 1), (40, 4, 4), (300, 130, 3)])
def test_route_tokens_sorts_the_pairs_by_expert(T, E, top):
    hip, _ = tables(torch.float32)
    g = torch.Generator().manual_seed(10)
    logits = torch.randn(T, E + 3, generator=g)
    logits[0, :2] = logits[0, :E].max() + 1.0                        # a tie: the lower index first
    r = hip.route_tokens(logits.to(DEV), E, top)
    best = torch.topk(logits[:, :E], top, dim=-1)
    chosen = r.chosen.cpu()
    assert torch.equal(chosen[1:].long(), best.indices[1:])
    assert chosen[0, 0] == 0 and (top == 1 or chosen[0, 1] == 1)
    close(r.shares, torch.softmax(torch.gather(logits, 1, chosen.long()), -1), 2e-6)
    order, place, tiles = r.order.cpu().long(), r.place_of.cpu().long(), r.tiles.cpu()
    assert sorted(order.tolist()) == list(range(T * top)) and torch.equal(order[place], torch.arange(T * top))
    by_row = chosen.reshape(-1)[order]
    assert torch.equal(by_row, torch.sort(by_row).values)               # an expert's rows lie together
    covered = []
    for e, row0, rows in tiles.tolist():
        if rows:
            assert 1 <= rows <= r.tile_rows and (by_row[row0:row0 + rows] == e).all()
            covered += list(range(row0, row0 + rows))
    assert covered == list(range(T * top))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,E,top,ff,K", [(1, 5, 2, 24, 64), (9, 12, 4, 64, 72), (150, 8, 3, 40, 96), (20, 3, 3, 8, 200),
                                          (9, 6, 2, 48, 64), (150, 8, 3, 80, 96), (400, 6, 2, 160, 128),
                                          (700, 4, 2, 192, 128), (900, 3, 3, 64, 320)])
def test_routed_experts(dtype, T, E, top, ff, K):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(T, K, generator=g).to(dtype)
    wgu = (torch.randn(E, 2 * ff, K, generator=g) * K ** -0.5).to(dtype)
    wd = (torch.randn(E, K, ff, generator=g) * ff ** -0.5).to(dtype)
    base = torch.randn(T, K, generator=g).to(dtype)
    logits = torch.randn(T, E, generator=g)
    r = hip.route_tokens(logits.to(DEV), E, top)
    for b in (base, None):
        got = hip.routed_experts(x.to(DEV), r, wgu.to(DEV), wd.to(DEV), None if b is None else b.to(DEV))
        want = emu.routed_experts(x, (r.chosen.cpu(), r.shares.cpu()), wgu, wd, b)
        close(got, want, 3e-6 if dtype == torch.float32 else 1.2e-2)
        tiled = (hip.prepare_expert_matrices(wgu.to(DEV), gated=True), hip.prepare_expert_matrices(wd.to(DEV)))
        assert tiled[0].tiled == (dtype == torch.bfloat16 and ff % 16 == 0 and K % 32 == 0)
        again = hip.routed_experts(x.to(DEV), r, tiled[0], tiled[1], None if b is None else b.to(DEV))
        assert torch.equal(again, got)                    # the same sums in the same order, from another layout
