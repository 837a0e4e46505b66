"""The Vevapel architecture as data: VevapelConfig -> ModelSpec.

A decoder with a layer norm (weight and bias) in front of AND behind every sublayer, the normed result added
times a constant ("sandwich" blocks); a scaled token embedding whose table is also the output head; three
mixers: grouped-query attention without rotation, with biases, a norm over the whole query and key projections,
queries that grow with the logarithm of the position and a gate per head ("gated_attention"); differential
attention, two score maps per head over the same values, rotated on part of each map's dims, seen through a
chunked mask, with a norm per head and a gate per element (the same part with `maps=2`); and the gated delta rule
with one decay per head and full-rank decay and gate projections ("channel_delta" with its options); routed
experts of gated units whose weights are the softmax over the chosen logits ("routed_moe" with its options); and
a run of layers that is repeated with the same weights, each pass with caches and states of its own, entered
through a product over [x ; embedding output] plus a vector per pass ("loop_join" ahead of the pass's first run).
Tensor names: `embed`, `loop.in|step`, `l<i>.norm1|norm1b|norm2|norm2b` (+ `.b`), `l<i>.mix.*`, `l<i>.mlp.e<j>.gate|up|down`,
`l<i>.mlp.router` (+ `.b`), `final.norm` (+ `.b`).
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.spec import LayerSpec, ModelSpec, PartSpec, PlanEntry
from ..config.vevapel import DeltaConfig, DiffAttentionConfig, GatedAttentionConfig, VevapelConfig


def _mixer_spec(cfg: VevapelConfig, m) -> PartSpec:
    common = {"hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
              "value_dim": m.vdim, "eps": cfg.norm_eps}
    if isinstance(m, DeltaConfig):
        return PartSpec("channel_delta", dict(common, conv_taps=m.conv, decay_rank=0, gate_rank=0, decay="head",
                                              gate="silu"), "mix")
    if isinstance(m, GatedAttentionConfig):
        return PartSpec("gated_attention", dict(common, scale=m.scale, bias=True, out_bias=True, qk_norm="whole",
                                                q_temp=(m.temp_coef, m.temp_every) if m.temp_every else None,
                                                gate="head"), "mix")
    assert isinstance(m, DiffAttentionConfig)
    position = {"kind": "none"}
    if m.rot_dims:
        position = {"kind": "rotary", "head_dim": m.dim, "rotary_dim": m.rot_dims, "theta": m.rot_base,
                    "max_position": cfg.max_position, "pairing": "half"}
    return PartSpec("gated_attention", dict(common, scale=m.scale, bias=True, out_bias=False, position=position,
                                            chunk=m.chunk, maps=2, diff=m.diff, sub_norm=True, out_scale=1.0 - m.diff,
                                            gate="element"), "mix")


def _mlp_spec(cfg: VevapelConfig, mlp) -> PartSpec:
    return PartSpec("routed_moe", {"hidden_size": cfg.width, "num_experts": mlp.experts, "top": mlp.top,
                                   "intermediate_size": mlp.ff, "activation": "swiglu", "router_bias": True}, "mlp")


def build_vevapel_spec(cfg: VevapelConfig) -> ModelSpec:
    norm = PartSpec("layernorm", {"hidden_size": cfg.width, "eps": cfg.norm_eps, "weight_name": "", "bias_name": "b"})
    layers = []
    for i, layer in enumerate(cfg.layers):
        parts = {"mixer_norm": norm.named("norm1"), "mixer": _mixer_spec(cfg, layer.mixer),
                 "mixer_out_norm": norm.named("norm1b")}
        if layer.mlp is not None:
            parts.update(ffn_norm=norm.named("norm2"), ffn=_mlp_spec(cfg, layer.mlp), ffn_out_norm=norm.named("norm2b"))
        layers.append(LayerSpec(f"l{i}", "sandwich", parts, {"mult": cfg.residual_mult}))
    plan = tuple(PlanEntry(i, before=None if turn is None else (0, turn)) for i, turn in cfg.run_order())
    stream_parts = ()
    if cfg.loop is not None:
        stream_parts = (PartSpec("loop_join", {"hidden_size": cfg.width, "times": cfg.loop.times}, "loop"),)
    sizes = {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "weight_name": ""}
    ignorable = []
    for i, layer in enumerate(cfg.layers):       # norms a checkpoint may carry for a layer without feed-forward
        if layer.mlp is None:
            ignorable += [f"l{i}.norm2", f"l{i}.norm2.b", f"l{i}.norm2b", f"l{i}.norm2b.b"]
    return ModelSpec(
        architecture="Vevapel",
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        max_position=cfg.max_position,
        embedding=PartSpec("token_embedding", dict(sizes, scale=cfg.embedding_scale), "embed"),
        layers=tuple(layers),
        plan=plan,
        final_norm=norm.named("final.norm"),
        # the output head is the embedding table itself, without the embedding's scale
        lm_head=PartSpec("lm_head", dict(sizes, tied_to="embed", tied_exact=True), "head"),
        eos_token_ids=cfg.eos_token_ids,
        ignorable_tensors=tuple(ignorable),
        stream_parts=stream_parts,
    )


register_architecture("Vevapel", VevapelConfig.from_dict, build_vevapel_spec)
