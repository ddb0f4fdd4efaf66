"""A state-space mixer: a decaying matrix state per head, fed through a short convolution, gated and normed.

With inner = heads * head_dim, N = state_size and G = groups, one product gives [z | x | B | C | dt] (inner, inner, G N,
G N, heads).  x, B and C together pass a causal convolution over time on every channel (`conv_taps` taps with a bias,
zeros before the sequence) and SiLU.  Per head h (using B and C of group h // (heads / G)):

    d_t = softplus(dt_t + dt_bias_h)
    S_t = exp(-exp(A_log_h) d_t) S_(t-1) + d_t B_t x_t^T          (S is N x head_dim, zero before the sequence)
    y_t = S_t^T C_t + D_h x_t

The heads' y times silu(z) is divided, in `norm_groups` equal parts, by each part's root mean square, multiplied by a
gain and projected back.  Step sizes, decays, the state, y and the norm are float32; the product's and the
convolution's outputs are in the activation dtype.  What a sequence keeps between steps is S and the convolution's
last taps - 1 inputs, both float32 states by name; there is nothing per token, so a step costs the same at any length.
"""
from ..cache.store import StateSpec
from ..models.spec import TensorSpec
from ..registry import register_part
from .base import Mixer


class StateSpaceMixer(Mixer):
    def __init__(self, hidden_size, num_heads, head_dim, state_size, groups, conv_taps, norm_groups, norm_eps,
                 tensors=("in", "conv", "conv.b", "dt_bias", "A_log", "D", "norm", "o")):
        self.hidden_size, self.num_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        self.state_size, self.groups, self.taps = int(state_size), int(groups), int(conv_taps)
        self.norm_groups, self.norm_eps = int(norm_groups), float(norm_eps)
        if self.num_heads % self.groups:
            raise ValueError(f"{num_heads} heads are no multiple of {groups} groups")
        if self.inner % self.norm_groups:
            raise ValueError(f"{self.inner} channels cannot be normed in {norm_groups} equal parts")
        if self.taps < 1:
            raise ValueError(f"a convolution needs at least one tap, found {conv_taps}")
        self.names = dict(zip(("in", "conv", "conv_b", "dt_bias", "a_log", "skip", "norm", "o"), tensors))

    @property
    def inner(self):
        return self.num_heads * self.head_dim

    @property
    def conv_channels(self):
        return self.inner + 2 * self.groups * self.state_size

    def tensor_specs(self):
        n, d, h = self.names, self.hidden_size, self.num_heads
        return {n["in"]: TensorSpec((self.inner + self.conv_channels + h, d)),
                n["conv"]: TensorSpec((self.conv_channels, self.taps), init="norm"),
                n["conv_b"]: TensorSpec((self.conv_channels,), init="norm"),
                n["dt_bias"]: TensorSpec((h,), init="norm"), n["a_log"]: TensorSpec((h,), init="norm"),
                n["skip"]: TensorSpec((h,), init="gain"), n["norm"]: TensorSpec((self.inner,), init="gain"),
                n["o"]: TensorSpec((d, self.inner))}

    def state_specs(self):
        specs = {"ssm": StateSpec((self.num_heads, self.state_size, self.head_dim), "float32")}
        if self.taps > 1:
            specs["conv"] = StateSpec((self.taps - 1, self.conv_channels), "float32")
        return specs

    def bind(self, tensors, rt):
        self.rt = rt
        n = self.names
        import torch
        w_in = tensors[n["in"]]
        spare = -w_in.shape[0] % 8           # zero rows, so that a row of the product is whole 16-byte pieces: the
        if spare:                            # convolution then reads its columns of it eight elements a load
            w_in = torch.cat([w_in, w_in.new_zeros((spare, w_in.shape[1]))], dim=0)
        self.w_in = rt.matrix(w_in.contiguous())
        self.conv_t = tensors[n["conv"]].float().t().contiguous()          # [taps, channels]
        self.conv_b = tensors[n["conv_b"]].float().contiguous()
        self.dt_bias = tensors[n["dt_bias"]].float().contiguous()
        self.a_log = tensors[n["a_log"]].float().contiguous()
        self.skip = tensors[n["skip"]].float().contiguous()
        self.norm_gain = tensors[n["norm"]].float().contiguous()
        self.w_o = rt.matrix(tensors[n["o"]])

    def forward(self, ctx, x, site):
        ops = ctx.ops
        inner, ch = self.inner, self.conv_channels
        u = ops.linear(x, self.w_in, ctx.dtype)                            # [M, z | x B C | dt]
        conv_state = self.state(ctx, "conv") if self.taps > 1 else None
        xbc = ops.conv_act(u[:, inner:inner + ch], self.conv_t, self.conv_b, conv_state, ctx.slot_ids, ctx.cu_rows, ctx.row_seq,
                           activation="silu", one_row_each=ctx.mode == "decode")
        y = ops.ssd_scan(xbc, u[:, :inner], u[:, inner + ch:inner + ch + self.num_heads], self.dt_bias, self.a_log, self.skip, self.state(ctx, "ssm"),
                         ctx.slot_ids, ctx.cu_rows, ctx.max_count, self.num_heads, self.groups, self.state_size, self.head_dim)
        y = ops.rms_norm(y, self.norm_gain, self.norm_eps, ctx.dtype, groups=self.norm_groups)
        return ops.linear(y, self.w_o, ctx.dtype, defer=True)


register_part("mixer", "state_space", StateSpaceMixer)
