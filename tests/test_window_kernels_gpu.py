"""The kernels behind the window attention mixers, each alone against plain tensor code:
layer norm with its adds, products with one matrix per head, the per-head norms with the
cache write, the latent row with its rotated part, and the attention itself (window and
kept first tokens, distance bias, sink, gate, values out of the key rows, shares of the
keys), over shuffled pages whose unused neighbours hold NaN."""
import math
import random
from types import SimpleNamespace

import pytest
import torch

import plain_topelorn as plain

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module", params=DTYPES, ids=["float32", "bfloat16"])
def ops(request):
    from servelab_amd.kernels import HipOps
    return HipOps(request.param, "cuda:0")


def close(got, want, dtype, scale=1.0):
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    err = (got.double().cpu() - want.double().cpu()).abs().max().item()
    assert err <= tol * scale, f"max abs err {err}, bar {tol * scale}"


def dev(t, dtype=None):
    return t.to(device="cuda:0", dtype=dtype or t.dtype).contiguous()


@pytest.mark.parametrize("T,H", [(1, 64), (5, 72), (33, 256), (3, 2600)])
def test_add_layernorm(ops, T, H):
    g = torch.Generator().manual_seed(T * H)
    dt = ops.act_dtype
    resid = torch.randn(T, H, generator=g) * 3 + 1.5
    d1 = torch.randn(T, H, generator=g).to(dt)
    d2 = torch.randn(T, H, generator=g).to(dt)
    gain = 1 + 0.3 * torch.randn(H, generator=g)
    for deltas in (None, d1, (d1, d2)):
        r = dev(resid.clone())
        want_sum = resid.double()
        for d in ([] if deltas is None else [deltas] if torch.is_tensor(deltas) else deltas):
            want_sum = want_sum + d.double()
        arg = None if deltas is None else dev(deltas) if torch.is_tensor(deltas) else tuple(dev(d) for d in deltas)
        out = ops.add_layernorm(r, arg, dev(gain), 1e-5)
        close(r, want_sum, torch.float32)                       # the stream itself stays float32
        close(out, plain.layer_norm_gain(want_sum, gain.double(), 1e-5), dt)
        # selected rows: the stream is left alone
        rows = torch.tensor([T - 1, 0], dtype=torch.int32)
        r2 = dev(resid.clone())
        out2 = ops.add_layernorm(r2, arg, dev(gain), 1e-5, rows=dev(rows))
        assert torch.equal(r2.cpu(), resid)
        close(out2, plain.layer_norm_gain(want_sum, gain.double(), 1e-5)[rows.long()], dt)


@pytest.mark.parametrize("T,heads,N,K,pad,col", [
    (1, 3, 40, 16, 8, 5), (7, 2, 5, 33, 0, 5), (130, 4, 70, 24, 3, 5), (64, 1, 64, 64, 0, 5),
    # aligned heads with K in steps of 32 and N in steps of 16: the matrix cores in bfloat16
    (3, 5, 48, 32, 8, 8), (130, 2, 80, 96, 0, 0), (17, 3, 16, 64, 16, 16)])
def test_head_products(ops, T, heads, N, K, pad, col):
    g = torch.Generator().manual_seed(T + N)
    dt = ops.act_dtype
    x = torch.randn(T, col + heads * (K + pad), generator=g).to(dt)
    A = (torch.randn(heads, N, K, generator=g) / K ** 0.5).to(dt)
    want = torch.einsum("thk,hnk->thn", x[:, col:].view(T, heads, K + pad)[..., :K].double(), A.double())
    y = ops.head_products(dev(x), col, heads, K + pad, dev(A))
    close(y.view(T, heads, N), want, dt)
    # into columns of a wider buffer, which stays as it was elsewhere
    gap = 3 if col == 5 else 4
    wide = torch.full((T, 4 + heads * (N + gap)), 7.0).to(dt)
    out = ops.head_products(dev(x), col, heads, K + pad, dev(A), y=dev(wide), y_col=4, y_head=N + gap)
    got = out[:, 4:].view(T, heads, N + gap)
    close(got[..., :N], want, dt)
    assert (got[..., N:] == 7).all() and (out[:, :4] == 7).all()


def paged(seq_lens, page, nkv, Dk, Dv, dtype, gen, num_pages=None):
    """Block tables over shuffled pages; page 0 and every page nobody owns hold NaN."""
    need = sum(-(-n // page) for n in seq_lens)
    num_pages = num_pages or need + 3
    order = list(range(1, num_pages))
    random.Random(int(torch.randint(0, 1000, (1,), generator=gen))).shuffle(order)
    width = max(-(-n // page) for n in seq_lens) + 1
    tables = torch.zeros(len(seq_lens), width, dtype=torch.int32)
    at = 0
    for s, n in enumerate(seq_lens):
        for j in range(-(-n // page)):
            tables[s, j] = order[at]
            at += 1
    kc = torch.full((num_pages, nkv, page, Dk), float("nan")).to(dtype)
    vc = torch.full((num_pages, nkv, max(Dv, 0), page), float("nan")).to(dtype)
    return tables, kc, vc


def fill_pages(tables, kc, vc, keys, values, page):
    for s, k in enumerate(keys):                          # k [n, nkv, Dk]
        for r in range(k.shape[0]):
            pg = int(tables[s, r // page])
            kc[pg, :, r % page] = k[r].to(kc.dtype)
            if values is not None:
                vc[pg, :, :, r % page] = values[s][r].to(vc.dtype)


def plain_attention(q, keys, values, q_pos, scale, window, keep, slopes, sinks, gates):
    """q [n, H, Dk] at positions q_pos of a sequence with keys [L, G, Dk], values [L, G, Dv]."""
    H, G = q.shape[1], keys.shape[1]
    L = keys.shape[0]
    kh = keys.repeat_interleave(H // G, dim=1).double()
    vh = values.repeat_interleave(H // G, dim=1).double()
    sc = torch.einsum("ihd,jhd->hij", q.double(), kh) * scale
    i = torch.as_tensor(q_pos)[:, None]
    j = torch.arange(L)[None, :]
    if slopes is not None:
        sc = sc - slopes.double()[:, None, None] * (i - j).double()[None]
    vis = (j <= i) & ((i - j < (window or L + 1)) | (j < keep))
    p = plain.softmax_with_sink(sc, vis, None if sinks is None else sinks.double())
    out = torch.einsum("hij,jhd->ihd", p, vh)
    if gates is not None:
        out = out * torch.sigmoid(gates.double())[:, :, None]
    return out


def run_attention(ops, seqs, page, H, G, Dk, Dv, scale, window, keep, slopes, sinks, gated, in_keys, seed):
    """``seqs``: (cached tokens before this step, tokens of this step) per sequence; multi-token ones
    first.  Returns (kernel output, plain output) over all tokens of the step."""
    dt = ops.act_dtype
    g = torch.Generator().manual_seed(seed)
    lens = [a + b for a, b in seqs]
    tables, kc, vc = paged(lens, page, G, Dk, 0 if in_keys else Dv, dt, g)
    keys = [torch.randn(n, G, Dk, generator=g).to(dt) for n in lens]
    values = [k[..., :Dv] for k in keys] if in_keys else [torch.randn(n, G, Dv, generator=g).to(dt) for n in lens]
    fill_pages(tables, kc, vc, keys, None if in_keys else values, page)
    T = sum(b for _, b in seqs)
    q = (torch.randn(T, 3 + H * Dk + H, generator=g)).to(dt)        # [pad | q heads | gates]
    cu, pos, at = [0], [], 0
    want = []
    for s, (a, b) in enumerate(seqs):
        qs = q[at:at + b, 3:3 + H * Dk].reshape(b, H, Dk)
        gates = q[at:at + b, 3 + H * Dk:] if gated else None
        want.append(plain_attention(qs, keys[s], values[s], list(range(a, a + b)), scale, window, keep,
                                    slopes, sinks, gates))
        pos += list(range(a, a + b))
        at += b
        cu.append(at)
    batch = SimpleNamespace(cu_q=dev(torch.tensor(cu, dtype=torch.int32)),
                            positions=dev(torch.tensor(pos, dtype=torch.int32)), num_seqs=len(seqs),
                            num_tokens=T, max_q_len=max(b for _, b in seqs), max_ctx_len=max(lens))
    qd = dev(q)
    out = ops.window_attention(qd, 3, H, G, Dk, Dv, dev(kc), None if in_keys else dev(vc), page, dev(tables),
                               batch, scale, window, keep, None if slopes is None else dev(slopes),
                               None if sinks is None else dev(sinks), qd if gated else None, 3 + H * Dk)
    return out.view(T, H, Dv), torch.cat(want)


@pytest.mark.parametrize("page", [16, 32])
@pytest.mark.parametrize("H,G,Dk,Dv", [(4, 2, 24, 16), (3, 3, 40, 8), (6, 1, 16, 40), (20, 1, 12, 36),
                                       (4, 2, 32, 16), (6, 1, 96, 64), (8, 8, 64, 64)])
def test_window_attention_prompts_and_single_tokens(ops, page, H, G, Dk, Dv):
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)])
    sinks = torch.randn(H, generator=torch.Generator().manual_seed(H))
    # whole prompts, a portion deep in its sequence, portions of two tokens, single tokens; windows that
    # end inside the step's own tokens, at page borders, and before the kept tokens
    seqs = [(0, 70), (45, 19), (0, 2), (61, 2), (0, 1), (16, 1), (15, 1), (100, 1), (31, 1)]
    for window, keep in ((9, 3), (16, 0), (33, 17), (None, 0), (1, 1)):
        got, want = run_attention(ops, seqs, page, H, G, Dk, Dv, Dk ** -0.5, window, keep, slopes, sinks,
                                  True, False, seed=page + H)
        assert torch.isfinite(got).all()
        close(got, want, ops.act_dtype, scale=2.0)


def test_window_attention_without_extras_and_values_from_key_rows(ops):
    for in_keys, Dk, Dv in ((True, 48, 40), (True, 16, 16), (False, 8, 24), (True, 64, 48)):
        got, want = run_attention(ops, [(0, 40), (37, 5), (52, 1)], 16, 5, 1, Dk, Dv, 0.3, 13, 0, None, None,
                                  False, in_keys, seed=Dk)
        close(got, want, ops.act_dtype, scale=2.0)


def test_single_tokens_in_shares_of_their_keys(ops):
    """Contexts long enough that a step of single tokens cuts its keys into shares, with sequences so
    short that some shares are empty."""
    H, G = 4, 2
    sinks = torch.tensor([0.5, -1.0, 2.0, 0.0])
    slopes = torch.tensor([0.5, 0.25, 0.1, 0.01])
    seqs = [(1500, 1), (3, 1), (0, 1), (700, 1)]
    for Dk, Dv in ((16, 24), (32, 16)):
        for window, keep in ((None, 0), (1000, 5), (600, 40)):
            got, want = run_attention(ops, seqs, 16, H, G, Dk, Dv, 0.25, window, keep, slopes, sinks, True, False,
                                      seed=9)
            close(got, want, ops.act_dtype, scale=2.0)


@pytest.mark.parametrize("Dk,Dv", [(16, 8), (32, 16)])
def test_one_far_key_shows(ops, Dk, Dv):
    """One key is made to stand out for one query; the output is its value exactly when the window or the
    kept first tokens let it be seen.  Keys just inside and just outside, at page borders."""
    dt = ops.act_dtype
    H = G = 1
    page, W, keep = 16, 48, 5
    for q_at, key_at, seen in ((200, 153, True), (200, 152, False), (200, 4, True), (200, 5, False),
                               (63, 16, True), (64, 16, False), (47, 0, True), (300, 0, True), (175, 128, True),
                               (176, 128, False), (176, 127, False)):
        g = torch.Generator().manual_seed(q_at)
        n = q_at + 1
        keys = torch.randn(n, 1, Dk, generator=g) * 0.1
        values = torch.randn(n, 1, Dv, generator=g)
        qv = torch.randn(Dk, generator=g)
        qv = qv / qv.norm()
        keys[key_at, 0] = 60.0 * qv
        for cached, new in ((0, n), (q_at, 1), (q_at - 1, 2)):                # in a prompt, decoded, in a short portion
            tables, kc, vc = paged([n], page, 1, Dk, Dv, dt, g)
            fill_pages(tables, kc, vc, [keys], [values], page)
            q = torch.randn(new, Dk, generator=g) * 0.1
            q[-1] = qv
            batch = SimpleNamespace(cu_q=dev(torch.tensor([0, new], dtype=torch.int32)),
                                    positions=dev(torch.arange(cached, n, dtype=torch.int32)), num_seqs=1,
                                    num_tokens=new, max_q_len=new, max_ctx_len=n)
            out = ops.window_attention(dev(q, dt), 0, H, G, Dk, Dv, dev(kc), dev(vc), page, dev(tables), batch,
                                       1.0, W, keep)[-1].float().cpu()
            hit = (out - values[key_at, 0].to(dt).float()).abs().max().item() < 0.05
            assert hit == seen, (q_at, key_at, cached, new)


def test_headnorm_store(ops):
    dt = ops.act_dtype
    g = torch.Generator().manual_seed(4)
    T, H, G, Dk, Dv, page, pages = 9, 4, 2, 24, 16, 16, 5
    width = (H + G) * Dk + G * Dv + H
    buf = torch.randn(T, width, generator=g).to(dt)
    qg, kg = 1 + 0.2 * torch.randn(Dk, generator=g), 1 + 0.2 * torch.randn(Dk, generator=g)
    other = torch.randn(T, 6 + G * Dv, generator=g).to(dt)
    slots = torch.tensor(random.Random(1).sample(range(pages * page), T), dtype=torch.int32)
    for v_first, lam in ((None, 0.0), (other[:, 6:], 0.3)):
        kc = torch.zeros(pages, G, page, Dk).to(dt)
        vc = torch.zeros(pages, G, Dv, page).to(dt)
        b, kcd, vcd = dev(buf.clone()), dev(kc), dev(vc)
        od = dev(other)
        ops.headnorm_store(b, H, G, Dk, Dv, dev(qg), dev(kg), 1e-5, None if v_first is None else od[:, 6:], lam,
                           dev(slots), kcd, vcd, page)
        x = buf.double()
        q = plain.rms_norm_gain(x[:, :H * Dk].view(T, H, Dk), qg.double(), 1e-5)
        k = plain.rms_norm_gain(x[:, H * Dk:(H + G) * Dk].view(T, G, Dk), kg.double(), 1e-5)
        v = x[:, (H + G) * Dk:(H + G) * Dk + G * Dv]
        if v_first is not None:
            v = (1 - lam) * v + lam * v_first.double()
        close(b[:, :H * Dk].view(T, H, Dk), q, dt)
        assert torch.equal(b[:, H * Dk:].cpu(), buf[:, H * Dk:])          # k, v and the rest stay as they were
        for t in range(T):
            pg, off = int(slots[t]) // page, int(slots[t]) % page
            close(kcd[pg, :, off], k[t], dt)
            close(vcd[pg, :, :, off], v[t].view(G, Dv), dt)
        written = torch.zeros(pages * page, dtype=torch.bool)
        written[slots.long()] = True
        assert (kcd.cpu().permute(0, 2, 1, 3).reshape(pages * page, -1)[~written] == 0).all()


def test_latent_store(ops):
    dt = ops.act_dtype
    g = torch.Generator().manual_seed(5)
    T, H, D, R, C, rot, page, pages = 7, 3, 16, 12, 40, 8, 16, 4
    down = H * (D + R)
    buf = torch.randn(T, down + C + R + H, generator=g).to(dt)
    gain = 1 + 0.2 * torch.randn(C, generator=g)
    pos = torch.tensor([0, 1, 2, 50, 51, 1000, 7], dtype=torch.int32)
    inv = 1.0 / (300.0 ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))
    cos, sin = ops.rope_tables(dev(pos), dev(inv))
    slots = torch.tensor(random.Random(2).sample(range(pages * page), T), dtype=torch.int32)
    kc = dev(torch.zeros(pages, 1, page, C + R).to(dt))
    q_out = dev(torch.zeros(T, H * (C + R)).to(dt))
    ops.latent_store(dev(buf), H, D, R, C, down, rot, dev(gain), 1e-6, SimpleNamespace(cos=cos, sin=sin),
                     dev(slots), kc, page, q_out)
    x = buf.double()
    c = plain.rms_norm_gain(x[:, down:down + C], gain.double(), 1e-6)
    kr = plain.rotate_pairs(x[:, down + C:down + C + R], pos, 300.0, rot)
    qr = plain.rotate_pairs(x[:, :down].view(T, H, D + R)[..., D:], pos, 300.0, rot)
    rows = kc.view(pages * page, C + R)[slots.long()]
    close(rows[:, :C], c, dt)
    close(rows[:, C:], kr, dt)
    close(q_out.view(T, H, C + R)[..., C:], qr, dt)
    assert (q_out.view(T, H, C + R)[..., :C] == 0).all()
