"""Golepel as data: layers in the order config.json lists them.

A layer is x += norm1(mixer(x + conv1(x))), x += norm2(ff(x + conv2(x))): the norms (RMS over equal groups of the
row) stand on the sub-layers' outputs only; a short causal convolution stands in front of each sub-layer.  The mixer
is attention through a cached latent; a layer with `kv_from` runs on the cache of the layer it names.  The
feed-forward is a SiLU-gated layer, a mixture of experts, or absent.  The head is the embedding table, its logits
times logit_scale.  Tensor names: embed, final.norm, l<i>.norm1/.norm2/.canon1/.canon2, l<i>.mix.{q,dkv,dkv.norm,uk,uv,o},
l<i>.mlp.{gate,up,down} or l<i>.mlp.router and l<i>.mlp.e<k>.{gate,up,down}.
"""
from ..config.golepel import GolepelConfig
from ..registry import register_architecture
from .spec import LayerSpec, ModelSpec, ScheduleEntry


def build_spec(c: GolepelConfig) -> ModelSpec:
    D = c.hidden_size
    norm = ("rms_norm", {"size": D, "eps": c.norm_eps, "groups": c.norm_groups, "tensor": "", "init": "gain"})
    conv = ("causal_conv", {"size": D, "taps": c.canon_taps, "residual": True, "tensor": ""})
    layers, schedule = [], []
    for i, l in enumerate(c.layers):
        m, p = l.mixer, f"l{i}."
        mixer = ("latent_attention", {
            "hidden_size": D, "num_heads": m.heads, "nope_dim": m.dim, "rope_dim": m.rot_dim, "value_dim": m.vdim,
            "latent_rank": m.kv_rank, "scale": m.scale, "latent_eps": c.norm_eps, "own_latent": m.kv_from is None,
            "position": ("rope", {"rotary_dim": m.rot_dims, "theta": m.rot_base}) if m.rot_dims else ("none", {})})
        if l.mlp is None:
            ff = None
        elif l.mlp.kind == "dense":
            ff = ("gated_mlp", {"hidden_size": D, "intermediate_size": l.mlp.ff, "activation": "silu",
                                "tensors": ("gate", "up", "down")})
        else:
            ff = ("routed_experts", {"hidden_size": D, "intermediate_size": l.mlp.ff, "n_experts": l.mlp.experts,
                                     "top": l.mlp.top, "limit": l.mlp.limit, "gate_alpha": 1.702, "up_shift": 1.0,
                                     "renormalize": False})
        prefixes = {"mixer": p + "mix.", "post_mixer_norm": p + "norm1", "mixer_conv": p + "canon1"}
        if ff is not None:
            prefixes.update({"feed_forward": p + "mlp.", "post_ff_norm": p + "norm2", "ff_conv": p + "canon2"})
        layers.append(LayerSpec(block=("post_norm", {"input_conv": conv}), mixer=mixer, feed_forward=ff, norm=norm,
                                prefixes=prefixes))
        schedule.append(ScheduleEntry(i, cache_of=m.kv_from))
    return ModelSpec(
        architecture=c.architecture, hidden_size=D, vocab_size=c.vocab_size,
        embedding=("scaled_embedding", {"vocab_size": c.vocab_size, "hidden_size": D, "scale": 1.0, "tensor": ""}),
        embedding_prefix="embed", layers=layers, schedule=schedule,
        final_norm=norm, final_norm_prefix="final.norm",
        head=("linear_head", {"vocab_size": c.vocab_size, "hidden_size": D, "softcap": None, "scale": c.logit_scale,
                              "tensor": ""}),
        head_prefix="embed", stop_ids=())


register_architecture(GolepelConfig.architecture, GolepelConfig, build_spec)
