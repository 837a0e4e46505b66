"""The Gesutar architecture as data: GesutarConfig -> ModelSpec.

A pre-norm decoder (RMS norms) whose token embedding is scaled and joined by a second table looked up by a
hash of the token and the one before it ("pair_embedding": the previous token is per-request state); whose
mixers attend over cached latents in a sliding window, with queries projected directly, interleaved
rotation on the rotated part, a learned sink per head in the softmax and a sigmoid gate per element of
the concatenated heads ("latent_attention" with its options); and whose feed-forwards are routed experts
of the form down(relu(up h)^2), chosen through groups, plus a shared expert ("routed_moe").  Tensor names:
`embed`, `bigram`, `l<i>.norm1|norm2`, `l<i>.mix.q|dkv|dkv.norm|uk|uv|sink|g|o`,
`l<i>.mlp.e<j>.up|down`, `l<i>.mlp.router`, `l<i>.mlp.shared.up|down`, `final.norm`, `head`.
"""
from __future__ import annotations

from ..config.gesutar import GesutarConfig
from ..config.registry import register_architecture
from ..config.spec import LayerSpec, ModelSpec, PartSpec, PlanEntry


def _mixer_spec(cfg: GesutarConfig, m) -> PartSpec:
    position = {"kind": "none"}
    if m.rot_dim:
        position = {"kind": "rotary", "head_dim": m.rot_dim, "rotary_dim": m.rot_dims, "theta": m.rot_base,
                    "max_position": cfg.max_position, "pairing": "interleaved"}
    return PartSpec("latent_attention", {
        "hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim, "value_dim": m.vdim,
        "q_rank": 0, "kv_rank": m.kv_rank, "scale": m.scale, "eps": cfg.norm_eps, "position": position,
        "window": m.window, "sink": True, "gate": "element"}, "mix")


def _mlp_spec(cfg: GesutarConfig, mlp) -> PartSpec:
    shared = {"intermediate_size": mlp.shared_ff} if mlp.shared_ff else None
    return PartSpec("routed_moe", {"hidden_size": cfg.width, "num_experts": mlp.experts, "top": mlp.top,
                                   "intermediate_size": mlp.ff, "groups": mlp.groups, "keep": mlp.keep,
                                   "scale": mlp.scale, "activation": "relu2", "shared": shared}, "mlp")


def build_gesutar_spec(cfg: GesutarConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"hidden_size": cfg.width, "eps": cfg.norm_eps, "weight_name": ""})
    layers, plan = [], []
    for i, layer in enumerate(cfg.layers):
        parts = {"mixer_norm": norm.named("norm1"), "mixer": _mixer_spec(cfg, layer.mixer)}
        if layer.mlp is not None:
            parts["ffn_norm"] = norm.named("norm2")
            parts["ffn"] = _mlp_spec(cfg, layer.mlp)
        layers.append(LayerSpec(f"l{i}", "pre_norm", parts))
        plan.append(PlanEntry(i))
    sizes = {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "weight_name": ""}
    if cfg.bigram is not None:
        embedding = PartSpec("pair_embedding", dict(sizes, buckets=cfg.bigram.buckets, mul_prev=cfg.bigram.mul_prev,
                                                    mul_cur=cfg.bigram.mul_cur, scale=cfg.embedding_scale,
                                                    pairs_name="bigram"), "embed")
    else:
        embedding = PartSpec("token_embedding", dict(sizes, scale=cfg.embedding_scale), "embed")
    return ModelSpec(
        architecture="Gesutar",
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        max_position=cfg.max_position,
        embedding=embedding,
        layers=tuple(layers),
        plan=tuple(plan),
        final_norm=norm.named("final.norm"),
        lm_head=PartSpec("lm_head", sizes, "head"),
        eos_token_ids=cfg.eos_token_ids,
        # a layer without feed-forward has no use for a second norm, should a checkpoint carry one
        ignorable_tensors=tuple(f"l{i}.norm2" for i, layer in enumerate(cfg.layers) if layer.mlp is None),
    )


register_architecture("Gesutar", GesutarConfig.from_dict, build_gesutar_spec)
