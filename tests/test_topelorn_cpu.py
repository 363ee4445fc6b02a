"""Topelorn without a GPU: configuration, registry, declared tensors, cache needs, the
page bookkeeping of a window that keeps the first tokens, and the plain implementation's
own mechanisms against each other."""
import copy
import math

import pytest
import torch

import plain_topelorn as plain
from servelab_amd import ConfigError, load_config
from servelab_amd.cache import CacheManager
from servelab_amd.config import TopelornConfig, resolve_architecture
from servelab_amd.parts.base import PagedKVSpec
from servelab_amd.parts.model import build_model_spec
from servelab_amd.weights.loader import Checkpoint, check_tensors
from topelorn_models import MODELS, make_weights, tensor_shapes, write_folder


@pytest.mark.parametrize("which", sorted(MODELS))
def test_config_is_read_and_declares_the_checkpoints_tensors(tmp_path, which):
    raw = MODELS[which]
    folder, _ = write_folder(tmp_path, raw, seed=1, tag=which)
    cfg = load_config(folder)
    assert isinstance(cfg, TopelornConfig) and cfg.width == raw["width"] and cfg.vocab == raw["vocab"]
    assert len(cfg.layers) == len(raw["layers"])
    spec = build_model_spec(cfg)
    check_tensors({n: s.shape for n, s in spec.param_specs().items()}, Checkpoint(folder).shapes(),
                  optional=spec.optional_tensors)
    assert {n for n in spec.param_specs()} | set(spec.optional_tensors) == set(tensor_shapes(raw))
    assert TopelornConfig.from_hf(cfg.to_hf()).layers == cfg.layers


def test_registry_takes_the_architecture_string():
    assert resolve_architecture({"architecture": "Topelorn"}).name == "Topelorn"
    assert resolve_architecture({"architectures": ["Qwen2ForCausalLM"]}).name == "Qwen2ForCausalLM"
    with pytest.raises(ValueError):
        resolve_architecture({"architecture": "Nothing"})


def test_missing_and_impossible_keys_are_named():
    raw = copy.deepcopy(MODELS["A"])
    del raw["layers"][0]["mixer"]["vdim"]
    with pytest.raises(ConfigError, match="vdim"):
        TopelornConfig.from_hf(raw)
    raw = copy.deepcopy(MODELS["A"])
    raw["layers"][1]["type"] = "convolution"
    with pytest.raises(ConfigError, match="convolution"):
        TopelornConfig.from_hf(raw)
    raw = copy.deepcopy(MODELS["A"])
    raw["layers"][3]["mixer"]["vdim"] = 24                      # mixed values of another width
    with pytest.raises(ConfigError, match="v_mix"):
        TopelornConfig.from_hf(raw)
    raw = copy.deepcopy(MODELS["A"])
    raw["layers"][1]["mixer"]["rot"]["dims"] = 7
    with pytest.raises(ConfigError, match="rot"):
        TopelornConfig.from_hf(raw)


def test_cache_needs_follow_the_layers():
    spec = build_model_spec(TopelornConfig.from_hf(MODELS["A"]))
    streams = spec.stream_specs()
    assert streams[0] == PagedKVSpec(2, 24, 9, value_dim=16, keep_first=3) == streams[2]
    assert streams[1] == PagedKVSpec(1, 48, 13, value_dim=0)          # latent 40 + rotated 8, no values
    assert streams[3] == PagedKVSpec(2, 8, 40, value_dim=16, keep_first=0)
    # the first layer that mixes values gives, the later ones take
    roles = [block.mixer.value_mix for _, block in spec.layers if hasattr(block.mixer, "value_mix")]
    assert roles == ["give", "take", "take"]
    roles_b = [getattr(block.mixer, "value_mix", "-") for _, block in
               build_model_spec(TopelornConfig.from_hf(MODELS["B"])).layers]
    assert roles_b == ["-", None, "give", "take"]


@pytest.mark.parametrize("keep,window,page", [(3, 9, 4), (20, 17, 16), (0, 5, 4), (4, 6, 4), (5, 1, 4)])
def test_window_pages_go_back_but_kept_first_pages_stay(keep, window, page):
    m = CacheManager({0: PagedKVSpec(1, 8, window, value_dim=4, keep_first=keep)}, 64, page, 4)
    assert m.open("a")
    total = 0
    for step in (1, 2, 7, 1, 1, 30, 1, 1, 1, 13):
        total += step
        assert m.grow("a", total)
        m.commit("a", total)
        table = m.block_table(0, "a")
        for j, p in enumerate(table):
            first, last = j * page, j * page + page - 1
            seen_later = last > total - window or first < keep     # by a query at total or later
            assert (p >= 0) == seen_later, (total, j, table)
        m.check()
    m.close("a")
    assert m.page_groups[0].allocator.num_free == 64


# ------------------------------------------------ the plain implementation itself
def test_plain_window_mask_edges():
    v = plain.window_mask(12, 4, 2)
    assert v[9, 9] and v[9, 6] and not v[9, 5]                 # 9 - 6 = 3 < 4 <= 9 - 5
    assert v[9, 0] and v[9, 1] and not v[9, 2]                 # kept: j < 2
    assert not v[3, 4]


def test_plain_sink_takes_its_share():
    scores = torch.zeros(1, 1, 3, dtype=torch.float64)
    vis = torch.ones(1, 3, dtype=torch.bool)
    p = plain.softmax_with_sink(scores, vis, torch.tensor([math.log(3.0)], dtype=torch.float64))
    assert torch.allclose(p, torch.full((1, 1, 3), 1 / 6, dtype=torch.float64))
    assert torch.allclose(plain.softmax_with_sink(scores, vis).sum(), torch.tensor(1.0, dtype=torch.float64))


def test_plain_rotation_keeps_lengths_and_relative_angles():
    x = torch.randn(5, 2, 12, dtype=torch.float64)
    pos = torch.tensor([0, 1, 7, 100, 1000])
    y = plain.rotate_pairs(x, pos, 300.0, 8)
    assert torch.allclose(y[0], x[0]) and torch.equal(y[..., 8:], x[..., 8:])
    assert torch.allclose(y[..., :8].norm(dim=-1), x[..., :8].norm(dim=-1))
    a, b = torch.randn(1, 8, dtype=torch.float64), torch.randn(1, 8, dtype=torch.float64)
    def dot(p, q):
        return (plain.rotate_pairs(a, torch.tensor([p]), 300.0, 8) * plain.rotate_pairs(b, torch.tensor([q]), 300.0, 8)).sum()
    assert torch.allclose(dot(9, 4), dot(105, 100))


def test_plain_latent_attention_equals_its_form_in_the_latents_space():
    """score and output through Wuk^T q and Wuv (sum p c): the form the engine computes."""
    cfg = MODELS["C"]
    m = cfg["layers"][1]["mixer"]
    w = plain.sub({n: t.double() for n, t in make_weights(cfg, 3).items()}, "l1.mix.")
    T, eps = 19, cfg["norm"]["eps"]
    h = torch.randn(T, cfg["width"], dtype=torch.float64)
    want = plain.latent_attention(h, w, m, eps)
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ w["q"].T).view(T, H, D + R)
    down = h @ w["dkv"].T
    c = plain.rms_norm_gain(down[:, :C], w["dkv.norm"], eps)
    kr = plain.rotate_pairs(down[:, C:], pos, m["rot"]["base"], m["rot"]["dims"])
    qr = plain.rotate_pairs(q[..., D:], pos, m["rot"]["base"], m["rot"]["dims"])
    q_lat = torch.einsum("thd,hdc->thc", q[..., :D], w["uk"].view(H, D, C))
    scores = (torch.einsum("ihc,jc->hij", q_lat, c) + torch.einsum("ihr,jr->hij", qr, kr)) * m["scale"]
    p = plain.softmax_with_sink(scores, plain.window_mask(T, m["mask"]["size"]))
    o_lat = torch.einsum("hij,jc->ihc", p, c)
    o = torch.einsum("ihc,hvc->ihv", o_lat, w["uv"].view(H, Dv, C)) * torch.sigmoid(h @ w["g"].T)[:, :, None]
    assert torch.allclose(o.reshape(T, H * Dv) @ w["o"].T, want, atol=1e-10)
