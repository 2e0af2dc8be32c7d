"""Toy parts defined by the tests, registered from outside the framework: a mixer with a state of fixed size
per sequence, a mixer that keeps one tensor per token (in a window's ring), another position table, a feed-forward with a router over experts, a norm of another kind, and an
architecture that mixes them with the built-in parts (one layer has two kinds of norm and a SiLU-gated feed-forward).  They are no model of anyone's; they show that the framework's files need no change
for a new part."""
import dataclasses
import math

import torch

from trapetum_amd.cache import StateSpec, TokenSpec
from trapetum_amd.config.base import ModelConfig, key
from trapetum_amd.models.spec import LayerSpec, ModelSpec, ScheduleEntry, TensorSpec
from trapetum_amd.parts import FeedForward, Mixer, Norm, Position
from trapetum_amd.registry import build_part, register_architecture, register_part


class EmaMixer(Mixer):
    """state_t = decay * state_{t-1} + (1 - decay) * x_t per sequence; out_t = proj(state_t)."""

    def __init__(self, hidden_size, decay):
        self.hidden_size = hidden_size
        self.decay = float(decay)

    def tensor_specs(self):
        return {"proj.weight": TensorSpec((self.hidden_size, self.hidden_size)),
                "proj.bias": TensorSpec((self.hidden_size,), init="norm")}

    def cache_spec(self):
        return StateSpec((self.hidden_size,), "float32")

    def bind(self, tensors, rt):
        self.rt = rt
        self.w = rt.matrix(tensors["proj.weight"])
        self.b = tensors["proj.bias"].float().contiguous()

    def forward(self, ctx, x, site):
        state = site.state                                   # [slots, hidden] fp32, zero for a fresh slot
        out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        row = 0
        for slot, count in zip(ctx.slots, ctx.counts):       # a scan over each sequence's rows of this step
            s = state[slot]
            for r in range(row, row + count):
                s = self.decay * s + (1.0 - self.decay) * x[r].float()
                out[r] = s
            state[slot] = s
            row += count
        return ctx.ops.linear(out.to(ctx.dtype), self.w, ctx.dtype, bias=self.b)       # a projection with a bias


class WindowMeanMixer(Mixer):
    """Keeps ONE tensor per token, h_t = in_proj(x_t) of `mem` elements, for the last `window` tokens;
    out_t = out_proj(mean of h_s over the tokens s <= t with t - s < window).  It reads what earlier steps cached
    through the page table (a ring's rows where the window is shorter than the context), then caches its own rows."""

    def __init__(self, hidden_size, mem, window):
        self.hidden_size, self.mem, self.window = hidden_size, mem, int(window)

    def tensor_specs(self):
        return {"in_proj.weight": TensorSpec((self.mem, self.hidden_size)), "out_proj.weight": TensorSpec((self.hidden_size, self.mem))}

    def cache_spec(self):
        return TokenSpec.of(self.window, h=(self.mem,))

    def bind(self, tensors, rt):
        self.rt = rt
        self.w_in, self.w_out = rt.matrix(tensors["in_proj.weight"]), rt.matrix(tensors["out_proj.weight"])

    def forward(self, ctx, x, site):
        pool = site.tensor("h")                              # [pages, page, mem]
        table = ctx.page_table(site.group_index).long()
        page, cap, W = pool.shape[1], site.rows_cap, self.window
        h = ctx.ops.linear(x, self.w_in, ctx.dtype)
        out = torch.empty((x.shape[0], self.mem), dtype=torch.float32, device=x.device)
        row = 0
        for i, (start, count) in enumerate(zip(ctx.starts, ctx.counts)):
            lo = max(0, start - (W - 1))
            pos = torch.arange(lo, start, device=x.device)
            rows = pos % cap if cap else pos
            seen = torch.cat([pool[table[i][rows // page], rows % page], h[row:row + count]]).float()     # positions lo ..
            for r in range(count):
                p = start + r
                out[row + r] = seen[max(lo, p - W + 1) - lo:p - lo + 1].mean(0)
            for r in range(count):                           # the step's own rows, cached after they were read
                p = start + r
                if cap and p + cap < start + count:
                    continue                                 # a later row of this step lands on the same ring row
                rr = p % cap if cap else p
                pool[table[i][rr // page], rr % page] = h[row + r]
            row += count
        return ctx.ops.linear(out.to(ctx.dtype), self.w_out, ctx.dtype)


class SoftRoutedMLP(FeedForward):
    """A router over experts, each a built-in gated feed-forward: out = sum_e softmax(router(x))_e * expert_e(x).
    Every expert runs on every row (a soft mixture), so the result is continuous in x."""

    def __init__(self, hidden_size, intermediate_size, n_experts):
        self.hidden_size, self.n_experts = hidden_size, n_experts
        self.experts = [build_part("feed_forward", ("gated_mlp", {"hidden_size": hidden_size, "intermediate_size": intermediate_size,
                                                                   "activation": "gelu_tanh"})) for _ in range(n_experts)]

    def tensor_specs(self):
        specs = {"router.weight": TensorSpec((self.n_experts, self.hidden_size))}
        for e, part in enumerate(self.experts):
            specs.update({f"experts.{e}.{name}": spec for name, spec in part.tensor_specs().items()})
        return specs

    def bind(self, tensors, rt):
        self.rt = rt
        self.w_router = rt.matrix(tensors["router.weight"])
        for e, part in enumerate(self.experts):
            head = f"experts.{e}."
            part.bind({n[len(head):]: t for n, t in tensors.items() if n.startswith(head)}, rt)

    def forward(self, ctx, x):
        weights = torch.softmax(ctx.ops.linear(x, self.w_router, torch.float32), dim=-1)      # router logits in fp32
        out = None
        for e, part in enumerate(self.experts):
            y = ctx.ops.rows(part.forward(ctx, x), torch.float32).float() * weights[:, e:e + 1]
            out = y if out is None else out + y
        return out.to(ctx.dtype)


class CenteredNorm(Norm):
    """(x - mean) / sqrt(var + eps) * w + b: a norm with a shift, which no RMS kernel fuses (it exposes no `gain`), so
    a block calls it through `forward` around a plain add."""

    def __init__(self, size, eps):
        self.size, self.eps = size, float(eps)

    def tensor_specs(self):
        return {"weight": TensorSpec((self.size,), init="norm"), "bias": TensorSpec((self.size,), init="norm")}

    def bind(self, tensors, rt):
        self.rt = rt
        self.w, self.b = tensors["weight"].float(), tensors["bias"].float()

    def forward(self, ctx, x, out_dtype=None):
        x = x.float()
        c = x - x.mean(-1, keepdim=True)
        y = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + self.eps) * (1.0 + self.w) + self.b
        return y.to(out_dtype or ctx.dtype)


class SquaredPosition(Position):
    """Rotary frequencies d -> 1 / (1 + d)^2 over part of the head, turning neighbours (2d, 2d + 1) together: another
    table and the other pairing through the same interface."""
    pairing = "neighbours"

    def __init__(self, rotary_dim):
        self.rotary_dim = rotary_dim

    def inv_freq(self, device):
        d = torch.arange(self.rotary_dim // 2, dtype=torch.float32)
        return (1.0 / (1.0 + d) ** 2).to(device)


@dataclasses.dataclass
class ToyConfig(ModelConfig):
    architecture = "ToyEmaForCausalLM"
    n_layers: int = key("n_layers", "int")
    width: int = key("width", "int")
    heads: int = key("heads", "int")
    head_size: int = key("head_size", "int")
    ff_width: int = key("ff_width", "int")
    vocab: int = key("vocab", "int")
    eps: float = key("eps", "float")
    decay: float = key("decay", "float")
    rotary: int = key("rotary", "int")
    experts: int = key("experts", "int")
    mem: int = key("mem", "int")
    mem_window: int = key("mem_window", "int")


def toy_spec(c):
    norm = ("rms_norm", {"size": c.width, "eps": c.eps, "weight_offset": 0.0})
    layers = []
    for l in range(c.n_layers):
        p = f"blocks.{l}."
        if l == 2:
            mixer = ("toy_window_mean", {"hidden_size": c.width, "mem": c.mem, "window": c.mem_window})
        elif l % 2 == 0:
            mixer = ("toy_ema", {"hidden_size": c.width, "decay": c.decay})
        else:
            mixer = ("attention", {"hidden_size": c.width, "num_heads": c.heads, "num_kv_heads": c.heads,
                                   "head_dim": c.head_size, "query_scale": 1.0 / math.sqrt(c.head_size),
                                   "position": ("toy_squared", {"rotary_dim": c.rotary})})
        norms = None
        if l == 2:
            ff = ("gated_mlp", {"hidden_size": c.width, "intermediate_size": c.ff_width, "activation": "gelu_tanh"})
        elif l % 2 == 0:    # a SiLU gate, and a second kind of norm in front of it
            ff = ("gated_mlp", {"hidden_size": c.width, "intermediate_size": c.ff_width, "activation": "silu"})
            norms = {"pre_ff_norm": ("toy_centered_norm", {"size": c.width, "eps": c.eps})}
        else:
            ff = ("toy_soft_routed", {"hidden_size": c.width, "intermediate_size": c.ff_width, "n_experts": c.experts})
        layers.append(LayerSpec(block=("pre_norm", {}), mixer=mixer, feed_forward=ff, norm=norm, norms=norms,
                                prefixes={"pre_mixer_norm": p + "n1.", "mixer": p + "mix.", "pre_ff_norm": p + "n2.",
                                          "feed_forward": p + "ff."}))
    # the order of running is data: layer 0 runs twice (its second run keeps a state of its own), and the
    # last entry runs the attention layer again on the cache its first run filled
    schedule = [ScheduleEntry(l) for l in range(c.n_layers)] + [ScheduleEntry(0), ScheduleEntry(1, cache_of=1)]
    return ModelSpec(architecture=c.architecture, hidden_size=c.width, vocab_size=c.vocab,
                     embedding=("scaled_embedding", {"vocab_size": c.vocab, "hidden_size": c.width, "scale": 1.0}),
                     embedding_prefix="emb.", layers=layers, schedule=schedule, final_norm=norm, final_norm_prefix="out_norm.",
                     head=("linear_head", {"vocab_size": c.vocab, "hidden_size": c.width, "softcap": None}),
                     head_prefix="head.")


def register():
    register_part("mixer", "toy_ema", EmaMixer)
    register_part("mixer", "toy_window_mean", WindowMeanMixer)
    register_part("position", "toy_squared", SquaredPosition)
    register_part("norm", "toy_centered_norm", CenteredNorm)
    register_part("feed_forward", "toy_soft_routed", SoftRoutedMLP)
    register_architecture(ToyConfig.architecture, ToyConfig, toy_spec)


TOY = dict(n_layers=3, width=48, heads=3, head_size=16, ff_width=80, vocab=97, eps=1e-5, decay=0.8, rotary=8, experts=3,
           mem=24, mem_window=11)


# ---- the toy's own plain reference: whole sequences, float64, no cache ------------------------------------------------
def toy_reference(cfg, W, tokens):
    D = torch.float64
    W = {k: v.to(D) for k, v in W.items()}
    T = len(tokens)
    x = W["emb.weight"][torch.tensor(tokens)]

    def norm(t, w):
        return t * torch.rsqrt((t * t).mean(-1, keepdim=True) + cfg["eps"]) * w

    def gelu(g):
        return 0.5 * g * (1 + torch.tanh(0.7978845608 * (g + 0.044715 * g ** 3)))

    def ema(t, p):
        s = torch.zeros(cfg["width"], dtype=D)
        out = []
        for r in range(T):
            s = cfg["decay"] * s + (1 - cfg["decay"]) * t[r]
            out.append(s)
        return torch.stack(out) @ W[p + "mix.proj.weight"].T + W[p + "mix.proj.bias"]

    def attn(t, p, kv=None):
        H, hd, rot = cfg["heads"], cfg["head_size"], cfg["rotary"]
        inv = 1.0 / (1.0 + torch.arange(rot // 2, dtype=D)) ** 2
        ang = torch.arange(T, dtype=D)[:, None] * inv[None]
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]

        def rope(u):                                       # neighbours turn together: pair d is elements 2d and 2d + 1
            u = u.reshape(T, H, hd)
            a, b = u[..., 0:rot:2], u[..., 1:rot:2]
            turned = torch.stack([a * c - b * s, b * c + a * s], -1).reshape(T, H, rot)
            return torch.cat([turned, u[..., rot:]], -1)
        q = rope(t @ W[p + "mix.q_proj.weight"].T)
        if kv is None:
            kv = (rope(t @ W[p + "mix.k_proj.weight"].T), (t @ W[p + "mix.v_proj.weight"].T).reshape(T, H, hd))
        k, v = kv
        sc = torch.einsum("thd,shd->hts", q, k) / math.sqrt(hd)
        sc = sc.masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool)), float("-inf"))
        o = torch.einsum("hts,shd->thd", torch.softmax(sc, -1), v).reshape(T, H * hd)
        return o @ W[p + "mix.o_proj.weight"].T, kv

    def window_mean(t, p):
        h = t @ W[p + "mix.in_proj.weight"].T
        m = torch.stack([h[max(0, r - cfg["mem_window"] + 1):r + 1].mean(0) for r in range(T)])
        return m @ W[p + "mix.out_proj.weight"].T

    kv1 = None
    for l, reuse in [(0, False), (1, False), (2, False), (0, False), (1, True)]:
        p = f"blocks.{l}."
        n = norm(x, W[p + "n1.weight"])
        if l == 0:
            x = x + ema(n, p)
        elif l == 2:
            x = x + window_mean(n, p)
        else:
            a, kv = attn(n, p, kv1 if reuse else None)
            kv1 = kv1 or kv
            x = x + a
        if l == 0:
            c = x - x.mean(-1, keepdim=True)
            n = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + cfg["eps"]) * (1 + W[p + "n2.weight"]) + W[p + "n2.bias"]
        else:
            n = norm(x, W[p + "n2.weight"])

        def mlp(t, q, act=gelu):
            return (act(t @ W[q + "gate_proj.weight"].T) * (t @ W[q + "up_proj.weight"].T)) @ W[q + "down_proj.weight"].T
        if l == 0:
            x = x + mlp(n, p + "ff.", lambda g: g * torch.sigmoid(g))
        elif l == 2:
            x = x + mlp(n, p + "ff.")
        else:
            mix = torch.softmax(n @ W[p + "ff.router.weight"].T, -1)
            x = x + sum(mix[:, e:e + 1] * mlp(n, p + f"ff.experts.{e}.") for e in range(cfg["experts"]))
    return norm(x, W["out_norm.weight"]) @ W["head.weight"].T
