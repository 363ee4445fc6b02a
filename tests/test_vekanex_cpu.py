"""Vekanex without a GPU: configuration and registry, declared tensors against a written
checkpoint, cache needs, the plain implementation's own mechanisms, and the engine's host side
(state slots, run list, batching, replay) over the kernel calls emulated in torch."""
import copy
import json
import random

import pytest
import torch

import plain_vekanex as plain
import replay_schedules as rs
from emulated_ops import EmulatedOps
from replay_harness import compare, replay_in_process
from servelab_amd import ConfigError, load_config
from servelab_amd.config import VekanexConfig, resolve_architecture
from servelab_amd.parts import PagedKVSpec, StateSpec
from servelab_amd.parts.model import build_model_spec
from servelab_amd.weights.loader import Checkpoint, check_tensors
from vekanex_models import MODELS, make_weights, tensor_shapes, write_folder

F = torch.float64


def make_requests(vocab, lengths, seed):
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


def reference(cfg, weights, requests):
    return {rid: plain.forward(cfg, weights, toks).float().numpy() for rid, toks in requests.items()}


# ------------------------------------------------------------------ configuration
@pytest.mark.parametrize("which", sorted(MODELS))
def test_config_round_trip_and_declared_tensors(tmp_path, which):
    cfg = MODELS[which]
    folder, _ = write_folder(tmp_path, cfg, seed=1, tag=which)
    assert resolve_architecture(json.load(open(folder + "/config.json"))).name == "Vekanex"
    config = load_config(folder)                      # low-rank widths come from the tensors' shapes
    assert isinstance(config, VekanexConfig)
    again = VekanexConfig.from_hf(config.to_hf())     # and travel as keys from then on
    assert again.layers == config.layers and again.to_hf() == config.to_hf()
    spec = build_model_spec(config)
    check_tensors({n: s.shape for n, s in spec.param_specs().items()}, Checkpoint(folder).shapes())
    assert {n: tuple(s.shape) for n, s in spec.param_specs().items()} == tensor_shapes(cfg)


def test_missing_and_impossible_keys_name_themselves():
    base = MODELS["A"]
    for path, text in ((("width",), "width"), (("norm",), "norm"),
                       (("layers", 1, "mixer", "gate_cap"), "gate_cap"),
                       (("layers", 2, "mixer", "tau"), "tau"),
                       (("layers", 0, "mixer", "left", "rot"), "rot"),
                       (("layers", 0, "mixer", "right", "conv"), "conv"),
                       (("layers", 0, "mlp", "router", "top"), "top")):
        cfg = copy.deepcopy(base)
        node = cfg
        for k in path[:-1]:
            node = node[k]
        del node[path[-1]]
        if path[0] == "layers":
            for l in cfg["layers"]:
                l.pop("weights_of", None)
        with pytest.raises(ConfigError, match=text):
            VekanexConfig.from_hf(cfg)
    cfg = copy.deepcopy(base)
    cfg["layers"][2]["mixer"].pop("decay_rank")       # no key and no checkpoint to read it from
    with pytest.raises(ConfigError, match="decay_rank"):
        VekanexConfig.from_hf(cfg)
    cfg = copy.deepcopy(base)
    cfg["layers"][3]["weights_of"] = 3
    with pytest.raises(ConfigError, match="weights_of"):
        VekanexConfig.from_hf(cfg)
    cfg = copy.deepcopy(base)
    cfg["layers"][3]["mixer"]["left_scale"] = 9.0     # describes another layer than the one it borrows
    with pytest.raises(ConfigError, match="another layer"):
        VekanexConfig.from_hf(cfg)
    cfg = copy.deepcopy(base)
    cfg["layers"][3]["weights_of"], cfg["layers"][0]["weights_of"] = 0, 3      # a ring: nobody has tensors
    with pytest.raises(ConfigError, match="weights_of"):
        VekanexConfig.from_hf(cfg)
    cfg = copy.deepcopy(base)
    cfg["layers"][1]["type"] = "rnn"
    with pytest.raises(ConfigError, match="mlstm, gla, parallel"):
        VekanexConfig.from_hf(cfg)


def test_borrowed_layers_and_keys_that_may_be_left_out():
    cfg = copy.deepcopy(MODELS["A"])
    cfg["layers"][4] = {"weights_of": 3}               # borrows from a borrower, and says nothing else
    del cfg["logit_softcap"], cfg["residual_mult"]
    got = VekanexConfig.from_hf(cfg)
    assert got.layers[4].weights_of == 0 and got.layers[4].mixer == got.layers[0].mixer
    assert got.layers[4].mlp == got.layers[0].mlp and got.layers[4].kind == "parallel"
    assert got.logit_softcap == 0.0 and got.residual_mult == 1.0
    spec = build_model_spec(got)
    assert [c.layer for c in spec.run] == [0, 1, 2, 0, 0] and spec.head[1].softcap is None


def test_cache_needs_and_run_list():
    spec = build_model_spec(VekanexConfig.from_hf(MODELS["A"]))
    assert len(spec.layers) == 3 and [c.layer for c in spec.run] == [0, 1, 2, 0, 2]
    needs = spec.stream_specs()
    assert len(needs) == 7                             # the parallel layers hold pages and a state each
    assert isinstance(needs[0], PagedKVSpec) and needs[0] == needs[4] and needs[0].v_dim == 24
    assert isinstance(needs[1], StateSpec) and needs[1] == needs[5]
    assert needs[1].shape == (4 * 16 * 8 + 3 * (2 * 2 * 16 + 4 * 8),)
    assert needs[2].shape == (3 * 8 * 16 + 3 * 8 + 3,) and needs[3].shape == (2 * 24 * 8,)


# ------------------------------------------------------------------ the plain implementation itself
def test_plain_gla_is_the_sum_over_decayed_keys():
    g = torch.Generator().manual_seed(0)
    T, w = 9, 16
    m = {"heads": 2, "dim": 4, "vdim": 3, "tau": 3.0}
    W = {n: torch.randn(s, generator=g, dtype=F) for n, s in
         {"q": (8, w), "k": (8, w), "v": (6, w), "g": (6, w), "o": (w, 6), "norm": (3,), "a1": (2, w),
          "a2": (8, 2), "a2.b": (8,)}.items()}
    h = torch.randn(T, w, generator=g, dtype=F)
    got = plain.gla(h, m, W, "", 1e-5)
    q = (h @ W["q"].T).view(T, 2, 4) * 0.5
    k, v = (h @ W["k"].T).view(T, 2, 4), (h @ W["v"].T).view(T, 2, 3)
    la = torch.log(torch.sigmoid((h @ W["a1"].T) @ W["a2"].T + W["a2.b"])).view(T, 2, 4) / 3.0
    o = torch.zeros(T, 2, 3, dtype=F)
    for t in range(T):
        for s in range(t + 1):
            decay = torch.exp(la[s + 1:t + 1].sum(0))                   # product of the decays after s
            o[t] += ((q[t] * decay * k[s]).sum(-1))[:, None] * v[s]
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-5) * W["norm"]
    gate = h @ W["g"].T
    want = (o.reshape(T, 6) * gate * torch.sigmoid(gate)) @ W["o"].T
    assert torch.allclose(got, want, atol=1e-10)


def test_plain_mlstm_is_the_unstabilised_recurrence():
    """With m taken out: C_t = sigmoid(f~) C + e^i k v^T, o = C^T q / (max(|n . q|, 1) + 1e-6 e^m)."""
    g = torch.Generator().manual_seed(1)
    T, w = 7, 12
    m = {"heads": 1, "dim": 3, "vdim": 2, "gate_cap": 5.0}
    W = {n: torch.randn(s, generator=g, dtype=F) for n, s in
         {"q": (3, w), "k": (3, w), "v": (2, w), "g": (2, w), "o": (w, 2), "norm": (2,), "i": (1, w),
          "i.b": (1,), "f": (1, w), "f.b": (1,)}.items()}
    h = torch.randn(T, w, generator=g, dtype=F)
    got = plain.mlstm(h, m, W, "", 1e-5)
    q, k, v = (h @ W["q"].T) * 3 ** -0.5, h @ W["k"].T, h @ W["v"].T
    ig = 5 * torch.tanh((h @ W["i"].T + W["i.b"]) / 5)[:, 0]
    fg = torch.log(torch.sigmoid(5 * torch.tanh((h @ W["f"].T + W["f.b"]) / 5)))[:, 0]
    C, n, mx, rows = torch.zeros(3, 2, dtype=F), torch.zeros(3, dtype=F), 0.0, []
    for t in range(T):
        C = torch.exp(fg[t]) * C + torch.exp(ig[t]) * k[t][:, None] * v[t][None, :]
        n = torch.exp(fg[t]) * n + torch.exp(ig[t]) * k[t]
        mx = max(float(fg[t]) + mx, float(ig[t]))
        scale = torch.exp(torch.tensor(mx, dtype=F))
        rows.append((C.T @ q[t]) / (torch.maximum((n @ q[t]).abs(), torch.tensor(1.0, dtype=F)) + 1e-6 * scale))
    o = torch.stack(rows)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-5) * W["norm"]
    want = (o * torch.sigmoid(h @ W["g"].T)) @ W["o"].T
    assert torch.allclose(got, want, atol=1e-9)


def test_plain_delta_rule_writes_what_it_reads():
    """With beta = 1 and no decay, reading with a token's own unit key returns its value."""
    cfgm = {"heads": 1, "kv_heads": 1, "dim": 4, "vdim": 3, "conv": 1}
    g = torch.Generator().manual_seed(2)
    T, w = 5, 8
    W = {n: torch.randn(s, generator=g, dtype=F) for n, s in
         {"q": (4, w), "k": (4, w), "v": (3, w), "a1": (2, w), "a2": (4, 2), "g1": (2, w), "g2": (3, 2),
          "o": (w, 3)}.items()}
    W.update({"q.conv": torch.ones(4, 1, dtype=F), "k.conv": torch.ones(4, 1, dtype=F),
              "v.conv": torch.ones(3, 1, dtype=F), "norm": torch.ones(3, dtype=F),
              "A_log": torch.full((1,), -40.0, dtype=F), "dt_bias": torch.zeros(4, dtype=F),
              "b": torch.zeros(1, w, dtype=F)})
    W["q"] = W["k"].clone()
    h = torch.randn(T, w, generator=g, dtype=F)
    # beta = sigmoid(0) = 1/2: after the write S^T k = v/2 + pred/2; check the recurrence by hand instead
    got = plain.gated_delta(h, cfgm, W, "", 1e-5)
    silu = lambda z: z * torch.sigmoid(z)
    k = silu(h @ W["k"].T)
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    v = silu(h @ W["v"].T)
    S, rows = torch.zeros(4, 3, dtype=F), []
    for t in range(T):
        S = S + 0.5 * k[t][:, None] * (v[t] - S.T @ k[t])[None, :]
        rows.append(S.T @ (k[t] * 0.5))
    o = torch.stack(rows)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-5)
    want = (o * torch.sigmoid((h @ W["g1"].T) @ W["g2"].T)) @ W["o"].T
    assert torch.allclose(got, want, atol=1e-9)


def test_plain_router_takes_the_largest_and_renormalises():
    w = {"router": torch.tensor([[1.0, 0], [0, 1.0], [-1.0, 0], [0.5, 0.5]], dtype=F)}
    for e in range(4):
        w[f"e{e}.gate"] = torch.full((2, 2), 10.0, dtype=F)
        w[f"e{e}.up"] = torch.eye(2, dtype=F) * (e + 1)
        w[f"e{e}.down"] = torch.eye(2, dtype=F)
    h = torch.tensor([[3.0, 1.0]], dtype=F)            # logits 3, 1, -3, 2: experts 0 and 3
    got = plain.routed_experts(h, {"router": {"experts": 4, "top": 2}}, w, "")
    share = torch.softmax(torch.tensor([3.0, 2.0], dtype=F), 0)
    act = plain.silu(torch.tensor([40.0, 40.0], dtype=F))
    assert torch.allclose(got[0], act * h[0] * (share[0] * 1 + share[1] * 4), atol=1e-9)


# ------------------------------------------------------------------ the engine's host side
@pytest.mark.parametrize("which", sorted(MODELS))
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "twos", "mixed"])
def test_every_way_of_cutting_gives_the_plain_logits(tmp_path, which, schedule):
    cfg = MODELS[which]
    folder, weights = write_folder(tmp_path, cfg, seed=11, tag=which)
    requests = make_requests(cfg["vocab"], [37, 1, 2, 49, 5, 26], seed=5)
    ref = reference(cfg, weights, requests)
    steps = {"whole": lambda: rs.whole(requests), "tail": lambda: rs.tail_decoded(requests, tail=12),
             "portions": lambda: rs.portions(requests),
             "twos": lambda: rs.portions(requests, sizes=(2, 2, 3, 2, 17, 2)),
             "mixed": lambda: rs.mixed(requests, {r: max(1, len(t) - 8) for r, t in requests.items()},
                                       max_live=3, seed=2)}[schedule]()
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, "float32", rs.max_tokens_needed(steps),
                      ops=EmulatedOps(torch.float32), device="cpu", max_live=3)
    worst, where = compare(out, steps, ref, cfg["vocab"])
    assert worst < 2e-4, f"max abs err {worst} at {where}"


def test_slots_that_held_another_request_start_from_zero(tmp_path):
    """Two slots, seven requests: every slot serves several requests, and what the last one left
    in it (state, last inputs of the convolution) must not reach the next."""
    cfg = MODELS["B"]
    folder, weights = write_folder(tmp_path, cfg, seed=12, tag="B")
    requests = make_requests(cfg["vocab"], [20, 3, 31, 1, 12, 2, 25], seed=6)
    ref = reference(cfg, weights, requests)
    steps = rs.mixed(requests, {r: len(t) // 2 for r, t in requests.items()}, max_live=2, seed=4,
                     max_portion=7)
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, "float32", rs.max_tokens_needed(steps),
                      ops=EmulatedOps(torch.float32), device="cpu", max_live=2)
    worst, where = compare(out, steps, ref, cfg["vocab"])
    assert worst < 2e-4, f"max abs err {worst} at {where}"
