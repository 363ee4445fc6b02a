"""Vekanex: a decoder whose config.json lists its layers, each a post-norm block.

    h += m * RMSNorm1(Mixer(h));  h += m * RMSNorm2(Experts(h))

The norms sit on the sublayers' outputs and the sublayers read the stream itself; m is
``residual_mult``.  The mixer is a matrix LSTM, a gated linear attention, or a softmax attention
beside a gated delta rule (``parts/recurrent.py``, ``parts/attention.py``); the feed-forward is a
set of routed experts with an optional shared one (``parts/routed.py``) or absent.  A layer with
``weights_of: j`` is a second call of block j in the run list, with cache streams of its own.
The final RMS norm is followed by a head of its own whose logits pass c * tanh(. / c).
Checkpoint names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
``final.norm``, ``head``.
"""
from ..config import VekanexConfig, register_architecture
from ..parts.attention import ProjectionNormAttention
from ..parts.block import PostNormBlock
from ..parts.embedding import OutputHead, TokenEmbedding
from ..parts.model import LayerCall, ModelSpec
from ..parts.norm import PostRMSNorm, RMSNorm
from ..parts.position import NoPosition, RotaryPosition
from ..parts.recurrent import GatedDeltaRule, GatedLinearAttention, MatrixLSTM, SideBySide
from ..parts.routed import RoutedExperts


def _mixer(cfg: VekanexConfig, layer):
    m, w, eps = layer.mixer, cfg.width, cfg.norm_eps
    if layer.kind == "mlstm":
        return MatrixLSTM(w, m.heads, m.dim, m.vdim, m.gate_cap, eps)
    if layer.kind == "gla":
        return GatedLinearAttention(w, m.heads, m.dim, m.vdim, m.tau, m.decay_rank, eps)
    a, b = m.left, m.right
    position = RotaryPosition(a.dim, a.rot_base, rotary_dim=a.rot_dims) if a.rot_dims else NoPosition()
    left = ProjectionNormAttention(w, a.heads, a.kv_heads, a.dim, a.vdim, a.scale, position, eps)
    right = GatedDeltaRule(w, b.heads, b.kv_heads, b.dim, b.vdim, b.conv, b.decay_rank, b.gate_rank, eps)
    return SideBySide(left, right, m.left_scale, m.right_scale)


def build_vekanex(cfg: VekanexConfig) -> ModelSpec:
    embedding = TokenEmbedding(cfg.vocab, cfg.width, name="embed")
    layers, block_of, run, streams = [], {}, [], 0
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is None:
            mlp = None
            if layer.mlp is not None:
                c = layer.mlp
                mlp = RoutedExperts(cfg.width, c.experts, c.top, c.ff, c.shared_ff)
            block = PostNormBlock(PostRMSNorm(cfg.width, cfg.norm_eps, cfg.residual_mult, name="norm1"),
                                  _mixer(cfg, layer),
                                  PostRMSNorm(cfg.width, cfg.norm_eps, cfg.residual_mult, name="norm2"),
                                  mlp, names=("", "mix.", "", "mlp."))
            block_of[i] = len(layers)
            layers.append((f"l{i}.", block))
    for i, layer in enumerate(cfg.layers):
        b = block_of[i if layer.weights_of is None else layer.weights_of]
        n = len(layers[b][1].cache_specs())
        run.append(LayerCall(b, tuple(range(streams, streams + n))))
        streams += n
    return ModelSpec(
        embedding=("", embedding),
        layers=layers,
        run=run,
        final_norm=("final.", RMSNorm(cfg.width, cfg.norm_eps, name="norm")),
        head=("", OutputHead(cfg.vocab, cfg.width, name="head", softcap=cfg.logit_softcap)),
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        eos_token_id=-1,
    )


register_architecture("Vekanex", VekanexConfig.from_hf, build_vekanex, model_type="vekanex")
