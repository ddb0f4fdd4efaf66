"""Lutovik as data: layers in the order config.json lists them.

A layer is x += n1b(mixer(n1(x))), x += n2b(ff(n2(x))) with RMS norms whose weight is stored around zero (gain 1 + w):
the `sandwich` block.  Mixers: grouped-query attention (values of their own size, rotation of neighbouring pairs on
the first rot.dims elements with frequencies scaled by wavelength; a layer with `kv_from` has no key and value
projections and runs on the cache of the layer it names), or `parallel`: an attention with split-half rotation and a
sigmoid gate on its heads beside a state-space mixer, their outputs normed and averaged.  Feed-forward: ReLU-gated, or
a mixture of SiLU-gated experts chosen by the largest sigmoid scores, each score scaling its expert's input, plus a
shared expert; or none.  The embedding is scaled; the head is a matrix of its own.
Tensor names: embed, head, final.norm, l<i>.norm1/.norm1b/.norm2/.norm2b, l<i>.mix.{q,k,v,o} or
l<i>.mix.left.{q,k,v,g,o,out} and l<i>.mix.right.{in,conv,conv.b,dt_bias,A_log,D,norm,o,out},
l<i>.mlp.{gate,up,down} or l<i>.mlp.router, l<i>.mlp.e<k>.{gate,up,down}, l<i>.mlp.shared.{gate,up,down}.
"""
from ..config.lutovik import LutovikConfig
from ..registry import register_architecture
from .spec import LayerSpec, ModelSpec, ScheduleEntry


def _attention(D, m, pairing, gate=False):
    position = ("rope", {"rotary_dim": m.rot.dims, "theta": m.rot.base, "pairing": pairing,
                         "scaling": m.rot.scaling_dict()}) if m.rot.dims else ("none", {})
    return ("attention", {"hidden_size": D, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                          "value_dim": m.vdim, "query_scale": m.scale, "position": position, "output_gate": gate,
                          "own_kv": m.kv_from is None, "precise_weights": True, "tensors": ("q", "k", "v", "o", "g")})


def build_spec(c: LutovikConfig) -> ModelSpec:
    D = c.hidden_size
    norm = ("rms_norm", {"size": D, "eps": c.norm_eps, "weight_offset": 1.0, "tensor": ""})
    layers, schedule = [], []
    for i, l in enumerate(c.layers):
        p = f"l{i}."
        if l.type == "attention":
            mixer, kv_from = _attention(D, l.mixer, "neighbours"), l.mixer.kv_from
        else:
            r = l.mixer.right
            right = ("state_space", {"hidden_size": D, "num_heads": r.heads, "head_dim": r.vdim, "state_size": r.state,
                                     "groups": r.groups, "conv_taps": r.conv, "norm_groups": r.norm_groups, "norm_eps": c.norm_eps})
            mixer = ("parallel", {"hidden_size": D, "left": _attention(D, l.mixer.left, "halves", gate=True), "right": right,
                                  "eps": c.norm_eps})
            kv_from = None
        if l.mlp is None:
            ff = None
        elif l.mlp.kind == "dense":
            ff = ("gated_mlp", {"hidden_size": D, "intermediate_size": l.mlp.ff, "activation": "relu",
                                "tensors": ("gate", "up", "down")})
        else:
            shared = None if l.mlp.shared_ff is None else (
                "gated_mlp", {"hidden_size": D, "intermediate_size": l.mlp.shared_ff, "activation": "silu",
                              "tensors": ("gate", "up", "down"), "prefix": "shared."})
            ff = ("routed_experts", {"hidden_size": D, "intermediate_size": l.mlp.ff, "n_experts": l.mlp.experts,
                                     "top": l.mlp.top, "limit": None, "gate_alpha": 1.0, "up_shift": 0.0,
                                     "renormalize": False, "score": "sigmoid", "weight_input": True, "shared": shared})
        prefixes = {"mixer": p + "mix.", "pre_mixer_norm": p + "norm1", "post_mixer_norm": p + "norm1b"}
        if ff is not None:
            prefixes.update({"feed_forward": p + "mlp.", "pre_ff_norm": p + "norm2", "post_ff_norm": p + "norm2b"})
        layers.append(LayerSpec(block=("sandwich", {}), mixer=mixer, feed_forward=ff, norm=norm, prefixes=prefixes))
        schedule.append(ScheduleEntry(i, cache_of=kv_from))
    return ModelSpec(
        architecture=c.architecture, hidden_size=D, vocab_size=c.vocab_size,
        embedding=("scaled_embedding", {"vocab_size": c.vocab_size, "hidden_size": D, "scale": c.embedding_scale, "tensor": ""}),
        embedding_prefix="embed", layers=layers, schedule=schedule,
        final_norm=norm, final_norm_prefix="final.norm",
        head=("linear_head", {"vocab_size": c.vocab_size, "hidden_size": D, "softcap": None, "tensor": ""}),
        head_prefix="head", stop_ids=())


register_architecture(LutovikConfig.architecture, LutovikConfig, build_spec)
