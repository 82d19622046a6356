"""Toy parts and toy architectures defined entirely in the tests and registered through the public registries;
nothing under tempura_amd/ knows about them.
* a mixer with per-request state of its own (a decaying running sum, no paged cache), used in some layers
  beside attention in others (``ToyForCausalLM``);
* a feed-forward with routing (each token goes to the expert its router scores highest) and a position
  encoding that is not rotary (a learned vector per position, added to queries and keys), in layers beside
  the library's own parts (``ToyRoutedForCausalLM``);
* a block arrangement with other parts than the library's: norms before AND after the mixer and the feed-forward
  (six named parts), and a second kind of layer that has a mixer and no feed-forward at all; and a norm that is not
  the library's (the mean taken out, a scale and a shift), at two of those sites and as the model's last norm
  (``ToySandwichForCausalLM``);
* a mixer whose pages hold something else than keys and values of heads: ONE compressed vector per token, declared
  by a cache spec of its own, in layers beside the library's attention (``ToyLatentForCausalLM``)."""
from __future__ import annotations

import json
from dataclasses import dataclass
from typing import Dict, List

import torch

from tempura_amd.config import LayerCall, LayerSpec, ModelSpec, PartSpec, register_architecture
from tempura_amd.parts import ArrangedBlock, CacheSpec, FeedForward, Mixer, Norm, PositionEncoding, StateSpec, WeightInfo, register_part


class DecaySumMixer(Mixer):
    """state <- decay * state + x W_in ; y = state W_out, token by token within each request."""

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.width = int(spec.params["width"])
        self.decay = float(spec.params["decay"])
        self.w_in = self.w_out = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        return {spec.weights["in"]: WeightInfo((spec.params["width"], hidden_size)),
                spec.weights["out"]: WeightInfo((hidden_size, spec.params["width"]))}

    def load_weights(self, get):
        self.w_in = self._to_device(get(self.spec.weights["in"]), torch.float32)
        self.w_out = self._to_device(get(self.spec.weights["out"]), torch.float32)

    def state_spec(self):
        return StateSpec((self.width,), torch.float32)

    def forward(self, x, ctx, cache, residual):
        u = x.float() @ self.w_in.T                                   # [tokens, width]
        for r in range(ctx.num_requests):
            slot, start, n = ctx.state_slot_list[r], ctx.q_starts[r], ctx.q_lens[r]
            s = cache.state[slot].clone()
            for t in range(start, start + n):
                s = self.decay * s + u[t]
                residual[t] += s @ self.w_out.T
            cache.state[slot] = s


register_part("mixer", "decay_sum", DecaySumMixer)


class DecaySumOnDeviceMixer(DecaySumMixer):
    """The same mixer, declared safe to capture: in a step of one token per request it finds its rows of the state
    through ``ctx.state_slots`` ON THE DEVICE (rows of a captured step that carry no request point at a spare row)
    and reads nothing on the host; steps with prompt portions, which are never captured, take the loop above."""
    graph_safe = True

    def forward(self, x, ctx, cache, residual):
        if ctx.max_q_len != 1:
            return super().forward(x, ctx, cache, residual)
        from tempura_amd.kernels import ops
        slots = ctx.state_slots.long()
        u = ops.linear(x.float().contiguous(), self.w_in, torch.float32)
        s = self.decay * cache.state.index_select(0, slots) + u
        cache.state.index_copy_(0, slots, s)
        ops.linear(s, self.w_out, torch.float32, residual=residual)


register_part("mixer", "decay_sum_on_device", DecaySumOnDeviceMixer)


class TopOneRoutedFFN(FeedForward):
    """Router logits in float32; each token's output is its best expert's two-layer ReLU network times the
    softmax weight of that expert.  Tokens are grouped by expert on the host; a token's result does not
    depend on which other tokens are in the batch."""

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.experts = int(spec.params["experts"])
        self.inner = int(spec.params["inner"])

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        e, i, w = spec.params["experts"], spec.params["inner"], spec.weights
        return {w["router"]: WeightInfo((e, hidden_size)), w["up"]: WeightInfo((e * i, hidden_size)),
                w["down"]: WeightInfo((e * hidden_size, i))}

    def load_weights(self, get):
        w = self.spec.weights
        self.router = self._to_device(get(w["router"]), torch.float32)
        self.up = self._to_device(get(w["up"]), torch.float32).view(self.experts, self.inner, self.hidden_size)
        self.down = self._to_device(get(w["down"]), torch.float32).view(self.experts, self.hidden_size, self.inner)

    def forward(self, x, ctx, residual):
        xf = x.float()
        probs = torch.softmax(xf @ self.router.T, dim=-1)
        weight, choice = probs.max(dim=-1)
        for e in range(self.experts):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                y = torch.relu(xf[rows] @ self.up[e].T) @ self.down[e].T
                residual[rows] += y * weight[rows, None]


class LearnedPosition(PositionEncoding):
    """A learned vector per position, added to every query and key head before the scores."""

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.table = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        return {spec.weights["table"]: WeightInfo((spec.params["max_positions"], spec.params["head_dim"]))}

    def load_weights(self, get):
        self.table = self._to_device(get(self.spec.weights["table"]), torch.float32)

    def apply(self, q, k, positions):
        d = self.table.shape[1]
        add = self.table[positions.long()]                                # [tokens, head_dim]
        q2 = (q.reshape(q.shape[0], -1, d) + add[:, None, :]).reshape(q.shape)
        k2 = None if k is None else (k.reshape(k.shape[0], -1, d) + add[:, None, :]).reshape(k.shape)
        return q2, k2


register_part("ffn", "toy_routed", TopOneRoutedFFN)
register_part("position", "toy_learned", LearnedPosition)


@dataclass
class ToyConfig:
    hidden_size: int = 48
    num_hidden_layers: int = 3
    vocab_size: int = 100
    width: int = 20
    decay: float = 0.8
    num_attention_heads: int = 4
    head_dim: int = 16
    intermediate_size: int = 64
    max_position_embeddings: int = 256
    state_on_device: bool = False       # the variant of the stateful mixer that may be captured in a graph
    architecture: str = "ToyForCausalLM"

    @classmethod
    def from_dict(cls, d):
        keys = cls.__dataclass_fields__
        return cls(**{k: v for k, v in d.items() if k in keys})

    def to_json(self):
        d = {k: getattr(self, k) for k in self.__dataclass_fields__}
        d["architectures"] = [self.architecture]
        return json.dumps(d)

    def build_spec(self) -> ModelSpec:
        layers = []
        for l in range(self.num_hidden_layers):
            p = f"toy.{l}"
            if l % 2 == 0:      # state layers at even depths, attention at odd ones
                mixer = PartSpec("decay_sum_on_device" if self.state_on_device else "decay_sum", {"width": self.width, "decay": self.decay},
                                 {"in": f"{p}.mix.in", "out": f"{p}.mix.out"})
            else:
                mixer = PartSpec("attention", {"num_heads": self.num_attention_heads, "num_kv_heads": 2,
                                               "head_dim": self.head_dim, "scale": self.head_dim ** -0.5, "window": None,
                                               "position": PartSpec("rope", {"head_dim": self.head_dim, "theta": 1e4, "scaling": None})},
                                 {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o"})
            layers.append(LayerSpec("prenorm", {
                "mixer": mixer,
                "ffn": PartSpec("swiglu", {"intermediate_size": self.intermediate_size},
                                {"gate": f"{p}.gate", "up": f"{p}.up", "down": f"{p}.down"}),
                "mixer_norm": PartSpec("rmsnorm", {"eps": 1e-5}, {"weight": f"{p}.n1"}),
                "ffn_norm": PartSpec("rmsnorm", {"eps": 1e-5}, {"weight": f"{p}.n2"})}))
        return ModelSpec(self.architecture, self.hidden_size, self.vocab_size, self.max_position_embeddings, layers,
                         [LayerCall(l) for l in range(self.num_hidden_layers)],
                         PartSpec("rmsnorm", {"eps": 1e-5}, {"weight": "toy.norm"}),
                         PartSpec("embedding", {}, {"weight": "toy.embed"}),
                         PartSpec("lm_head", {"tied": True, "tied_to": "toy.embed"}, {"weight": "toy.head"}))


register_architecture("ToyForCausalLM", ToyConfig)


@dataclass
class ToyRoutedConfig:
    """Three layers: attention with a learned position and a routed feed-forward; attention with rotary
    position (window 12) and the library's SwiGLU; again a learned position and a routed feed-forward."""
    hidden_size: int = 64
    vocab_size: int = 90
    num_attention_heads: int = 4
    num_key_value_heads: int = 2
    head_dim: int = 16
    experts: int = 3
    inner: int = 40
    intermediate_size: int = 96
    max_position_embeddings: int = 128
    architecture: str = "ToyRoutedForCausalLM"

    @classmethod
    def from_dict(cls, d):
        keys = cls.__dataclass_fields__
        return cls(**{k: v for k, v in d.items() if k in keys})

    def to_json(self):
        d = {k: getattr(self, k) for k in self.__dataclass_fields__}
        d["architectures"] = [self.architecture]
        return json.dumps(d)

    def _attention(self, p, position, window):
        return PartSpec("attention", {"num_heads": self.num_attention_heads, "num_kv_heads": self.num_key_value_heads,
                                      "head_dim": self.head_dim, "scale": self.head_dim ** -0.5, "window": window,
                                      "position": position},
                        {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o"})

    def build_spec(self) -> ModelSpec:
        learned = lambda p: PartSpec("toy_learned", {"max_positions": self.max_position_embeddings, "head_dim": self.head_dim},
                                     {"table": f"{p}.pos"})
        rope = PartSpec("rope", {"head_dim": self.head_dim, "theta": 1e4, "scaling": None})
        routed = lambda p: PartSpec("toy_routed", {"experts": self.experts, "inner": self.inner},
                                    {"router": f"{p}.router", "up": f"{p}.up", "down": f"{p}.down"})
        swiglu = lambda p: PartSpec("swiglu", {"intermediate_size": self.intermediate_size},
                                    {"gate": f"{p}.gate", "up": f"{p}.up", "down": f"{p}.down"})
        norm = lambda n: PartSpec("rmsnorm", {"eps": 1e-5}, {"weight": n})
        block = lambda mixer, ffn, n1, n2: LayerSpec("prenorm", {"mixer": mixer, "ffn": ffn, "mixer_norm": n1, "ffn_norm": n2})
        layers = [
            block(self._attention("r.0", learned("r.0"), None), routed("r.0"), norm("r.0.n1"), norm("r.0.n2")),
            block(self._attention("r.1", rope, 12), swiglu("r.1"), norm("r.1.n1"), norm("r.1.n2")),
            block(self._attention("r.2", learned("r.2"), None), routed("r.2"), norm("r.2.n1"), norm("r.2.n2")),
        ]
        return ModelSpec(self.architecture, self.hidden_size, self.vocab_size, self.max_position_embeddings, layers,
                         [LayerCall(0), LayerCall(1), LayerCall(2)],
                         norm("r.norm"), PartSpec("embedding", {}, {"weight": "r.embed"}),
                         PartSpec("lm_head", {"tied": False}, {"weight": "r.head"}))


register_architecture("ToyRoutedForCausalLM", ToyRoutedConfig)


def plain_routed_forward(cfg: ToyRoutedConfig, W: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    """Whole sequence, no cache, float64: the routed toy model written out plainly."""
    import plain
    W = {k: v.double() for k, v in W.items()}
    T = len(tokens)
    H, KV, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    h = W["r.embed"][torch.tensor(tokens)]
    inv = plain.rope_inv_freq(D, 1e4, None)
    pos = torch.arange(T)
    for l in range(3):
        p = f"r.{l}"
        x = plain.rmsnorm(h, W[f"{p}.n1"], 1e-5)
        q = (x @ W[f"{p}.q"].T).reshape(T, H, D)
        k = (x @ W[f"{p}.k"].T).reshape(T, KV, D)
        v = (x @ W[f"{p}.v"].T).reshape(T, KV, D)
        if l == 1:
            q, k = plain.rope(q, pos, inv), plain.rope(k, pos, inv)
            a = plain.attention(q, k, v, D ** -0.5, window=12)
        else:
            add = W[f"{p}.pos"][:T]
            q, k = q + add[:, None, :], k + add[:, None, :]
            a = plain.attention(q, k, v, D ** -0.5)
        h = h + a @ W[f"{p}.o"].T
        x = plain.rmsnorm(h, W[f"{p}.n2"], 1e-5)
        if l == 1:
            h = h + plain.swiglu_ffn(x, W[f"{p}.gate"], W[f"{p}.up"], W[f"{p}.down"])
        else:
            probs = torch.softmax(x @ W[f"{p}.router"].T, dim=-1)
            weight, choice = probs.max(dim=-1)
            up = W[f"{p}.up"].view(cfg.experts, cfg.inner, cfg.hidden_size)
            down = W[f"{p}.down"].view(cfg.experts, cfg.hidden_size, cfg.inner)
            y = torch.stack([torch.relu(x[t] @ up[choice[t]].T) @ down[choice[t]].T * weight[t] for t in range(T)])
            h = h + y
    return plain.rmsnorm(h, W["r.norm"], 1e-5) @ W["r.head"].T


def plain_toy_forward(cfg: ToyConfig, W: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    """Whole sequence, no cache, float64: the toy model written out plainly."""
    import plain
    W = {k: v.double() for k, v in W.items()}
    T = len(tokens)
    h = W["toy.embed"][torch.tensor(tokens)]
    inv = plain.rope_inv_freq(cfg.head_dim, 1e4, None)
    pos = torch.arange(T)
    for l in range(cfg.num_hidden_layers):
        p = f"toy.{l}"
        x = plain.rmsnorm(h, W[f"{p}.n1"], 1e-5)
        if l % 2 == 0:
            u = x @ W[f"{p}.mix.in"].T
            s = torch.zeros(cfg.width, dtype=torch.float64)
            ys = []
            for t in range(T):
                s = cfg.decay * s + u[t]
                ys.append(s @ W[f"{p}.mix.out"].T)
            h = h + torch.stack(ys)
        else:
            q = plain.rope((x @ W[f"{p}.q"].T).reshape(T, cfg.num_attention_heads, cfg.head_dim), pos, inv)
            k = plain.rope((x @ W[f"{p}.k"].T).reshape(T, 2, cfg.head_dim), pos, inv)
            v = (x @ W[f"{p}.v"].T).reshape(T, 2, cfg.head_dim)
            h = h + plain.attention(q, k, v, cfg.head_dim ** -0.5) @ W[f"{p}.o"].T
        x = plain.rmsnorm(h, W[f"{p}.n2"], 1e-5)
        h = h + plain.swiglu_ffn(x, W[f"{p}.gate"], W[f"{p}.up"], W[f"{p}.down"])
    return plain.rmsnorm(h, W["toy.norm"], 1e-5) @ W["toy.embed"].T


class CentredNorm(Norm):
    """y = (x - mean(x)) / sqrt(var(x) + eps) * scale + shift, in float32; two tensors."""

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.eps = float(spec.params["eps"])

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        return {spec.weights["scale"]: WeightInfo((hidden_size,), "ones"), spec.weights["shift"]: WeightInfo((hidden_size,))}

    def load_weights(self, get):
        self.scale = self._to_device(get(self.spec.weights["scale"]), torch.float32)
        self.shift = self._to_device(get(self.spec.weights["shift"]), torch.float32)

    def forward(self, h, rows=None):
        x = h if rows is None else h.index_select(0, rows.long())
        x = x - x.mean(dim=-1, keepdim=True)
        return (x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + self.eps) * self.scale + self.shift).to(self.dtype)


register_part("norm", "toy_centred", CentredNorm)


def plain_centred_norm(x, scale, shift, eps):
    x = x - x.mean(dim=-1, keepdim=True)
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * scale + shift


class SandwichBlock(ArrangedBlock):
    """h += post_mixer_norm(mixer(pre_mixer_norm(h))); h += post_ffn_norm(ffn(pre_ffn_norm(h))): six parts, two of
    them norms that the library's own arrangement does not have.  A part adds its result into the stream it is
    handed, so the block hands it a zero stream and norms what comes back."""
    ROLES = {"pre_mixer_norm": "norm", "mixer": "mixer", "post_mixer_norm": "norm",
             "pre_ffn_norm": "norm", "ffn": "ffn", "post_ffn_norm": "norm"}

    def forward(self, h, ctx, cache):
        y = torch.zeros_like(h)
        self.mixer.forward(self.pre_mixer_norm.forward(h), ctx, cache, y)
        h += self.post_mixer_norm.forward(y).float()
        y = torch.zeros_like(h)
        self.ffn.forward(self.pre_ffn_norm.forward(h), ctx, y)
        h += self.post_ffn_norm.forward(y).float()


class MixerOnlyBlock(ArrangedBlock):
    """h += mixer(norm(h)) and nothing else: a layer without a feed-forward."""
    ROLES = {"norm": "norm", "mixer": "mixer"}

    def forward(self, h, ctx, cache):
        self.mixer.forward(self.norm.forward(h), ctx, cache, h)


register_part("block", "toy_sandwich", SandwichBlock)
register_part("block", "toy_mixer_only", MixerOnlyBlock)


@dataclass
class ToySandwichConfig:
    """Layer 0: the sandwich arrangement around attention and SwiGLU; layer 1: attention alone; layer 2: sandwich."""
    hidden_size: int = 64
    vocab_size: int = 120
    num_attention_heads: int = 4
    num_key_value_heads: int = 2
    head_dim: int = 16
    intermediate_size: int = 96
    max_position_embeddings: int = 128
    architecture: str = "ToySandwichForCausalLM"

    @classmethod
    def from_dict(cls, d):
        keys = cls.__dataclass_fields__
        return cls(**{k: v for k, v in d.items() if k in keys})

    def to_json(self):
        d = {k: getattr(self, k) for k in self.__dataclass_fields__}
        d["architectures"] = [self.architecture]
        return json.dumps(d)

    def build_spec(self) -> ModelSpec:
        rope = PartSpec("rope", {"head_dim": self.head_dim, "theta": 1e4, "scaling": None})
        norm = lambda n: PartSpec("rmsnorm", {"eps": 1e-5}, {"weight": n})
        centred = lambda n: PartSpec("toy_centred", {"eps": 1e-4}, {"scale": n + ".scale", "shift": n + ".shift"})
        attn = lambda p: PartSpec("attention", {"num_heads": self.num_attention_heads, "num_kv_heads": self.num_key_value_heads,
                                                "head_dim": self.head_dim, "scale": self.head_dim ** -0.5, "window": None,
                                                "position": rope}, {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o"})
        swiglu = lambda p: PartSpec("swiglu", {"intermediate_size": self.intermediate_size},
                                    {"gate": f"{p}.gate", "up": f"{p}.up", "down": f"{p}.down"})
        # (the centred norm after the mixer and before the feed-forward of the sandwich layers, and as the last norm)
        sandwich = lambda p: LayerSpec("toy_sandwich", {
            "pre_mixer_norm": norm(f"{p}.n1"), "mixer": attn(p), "post_mixer_norm": centred(f"{p}.n2"),
            "pre_ffn_norm": centred(f"{p}.n3"), "ffn": swiglu(p), "post_ffn_norm": norm(f"{p}.n4")})
        layers = [sandwich("s.0"), LayerSpec("toy_mixer_only", {"norm": norm("s.1.n1"), "mixer": attn("s.1")}), sandwich("s.2")]
        return ModelSpec(self.architecture, self.hidden_size, self.vocab_size, self.max_position_embeddings, layers,
                         [LayerCall(0), LayerCall(1), LayerCall(2)], centred("s.norm"),
                         PartSpec("embedding", {}, {"weight": "s.embed"}), PartSpec("lm_head", {"tied": False}, {"weight": "s.head"}))


register_architecture("ToySandwichForCausalLM", ToySandwichConfig)


def plain_sandwich_forward(cfg: ToySandwichConfig, W: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    """Whole sequence, no cache, float64: the sandwich toy model written out plainly."""
    import plain
    W = {k: v.double() for k, v in W.items()}
    T = len(tokens)
    H, KV, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    h = W["s.embed"][torch.tensor(tokens)]
    inv = plain.rope_inv_freq(D, 1e4, None)
    pos = torch.arange(T)

    def attend(p, x):
        q = plain.rope((x @ W[f"{p}.q"].T).reshape(T, H, D), pos, inv)
        k = plain.rope((x @ W[f"{p}.k"].T).reshape(T, KV, D), pos, inv)
        v = (x @ W[f"{p}.v"].T).reshape(T, KV, D)
        return plain.attention(q, k, v, D ** -0.5) @ W[f"{p}.o"].T
    for l in range(3):
        p = f"s.{l}"
        if l == 1:
            h = h + attend(p, plain.rmsnorm(h, W[f"{p}.n1"], 1e-5))
            continue
        cn = lambda x, n: plain_centred_norm(x, W[n + ".scale"], W[n + ".shift"], 1e-4)
        h = h + cn(attend(p, plain.rmsnorm(h, W[f"{p}.n1"], 1e-5)), f"{p}.n2")
        y = plain.swiglu_ffn(cn(h, f"{p}.n3"), W[f"{p}.gate"], W[f"{p}.up"], W[f"{p}.down"])
        h = h + plain.rmsnorm(y, W[f"{p}.n4"], 1e-5)
    return plain_centred_norm(h, W["s.norm.scale"], W["s.norm.shift"], 1e-4) @ W["s.head"].T


# ---- a mixer with another per-token cache layout -------------------------------------------------------------------
@dataclass(frozen=True)
class LatentCacheSpec(CacheSpec):
    """A page holds ``page_size`` compressed vectors of ``latent`` elements and nothing else (no heads, no separate
    values): one plane, ``c``.  ``num_kv_heads`` and ``head_dim`` are not used."""
    latent: int = 0

    def planes(self, page_size):
        return {"c": (page_size, self.latent)}


class LatentMixer(Mixer):
    """c_t = x_t W_c is all a token leaves in the cache; token t's output is softmax_j<=t(q_t . c_j / sqrt(latent))
    applied to the c_j themselves, times W_out (q_t = x_t W_q)."""

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.latent = int(spec.params["latent"])

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        n, w = spec.params["latent"], spec.weights
        return {w["q"]: WeightInfo((n, hidden_size)), w["c"]: WeightInfo((n, hidden_size)), w["out"]: WeightInfo((hidden_size, n))}

    def load_weights(self, get):
        w = self.spec.weights
        self.wq, self.wc, self.wout = (self._to_device(get(w[k]), torch.float32) for k in ("q", "c", "out"))

    def cache_spec(self):
        return LatentCacheSpec("full", 1, self.latent, None, self.latent)

    def forward(self, x, ctx, cache, residual):
        xf = x.float()
        q, c = xf @ self.wq.T, xf @ self.wc.T
        pool = cache.planes["c"]                                          # [pages + 1, page_size, latent]
        ps = cache.page_size
        flat = pool.view(-1, self.latent)
        flat[ctx.slot_mapping[cache.group].long()] = c.to(pool.dtype)     # this step's vectors into their cache places
        tables = ctx.block_tables[cache.group].tolist()
        for r in range(ctx.num_requests):
            start, n, total = ctx.q_starts[r], ctx.q_lens[r], ctx.ctx_lens[r]
            rows = torch.tensor([tables[r][j // ps] * ps + j % ps for j in range(total)], device=flat.device)
            keys = flat[rows].float()                                     # every vector of the request, in order
            for i in range(n):
                upto = total - n + i + 1
                p = torch.softmax(keys[:upto] @ q[start + i] / self.latent ** 0.5, dim=0)
                residual[start + i] += (p @ keys[:upto]) @ self.wout.T


register_part("mixer", "toy_latent", LatentMixer)


@dataclass
class ToyLatentConfig:
    """Layers 0 and 2: the latent mixer; layer 1: the library's attention.  Two cache groups with different pages."""
    hidden_size: int = 48
    vocab_size: int = 110
    latent: int = 20
    num_attention_heads: int = 4
    num_key_value_heads: int = 2
    head_dim: int = 16
    intermediate_size: int = 64
    max_position_embeddings: int = 128
    architecture: str = "ToyLatentForCausalLM"

    @classmethod
    def from_dict(cls, d):
        keys = cls.__dataclass_fields__
        return cls(**{k: v for k, v in d.items() if k in keys})

    def to_json(self):
        d = {k: getattr(self, k) for k in self.__dataclass_fields__}
        d["architectures"] = [self.architecture]
        return json.dumps(d)

    def build_spec(self) -> ModelSpec:
        norm = lambda n: PartSpec("rmsnorm", {"eps": 1e-5}, {"weight": n})
        layers = []
        for l in range(3):
            p = f"z.{l}"
            if l == 1:
                mixer = PartSpec("attention", {"num_heads": self.num_attention_heads, "num_kv_heads": self.num_key_value_heads,
                                               "head_dim": self.head_dim, "scale": self.head_dim ** -0.5, "window": None,
                                               "position": PartSpec("rope", {"head_dim": self.head_dim, "theta": 1e4, "scaling": None})},
                                 {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o"})
            else:
                mixer = PartSpec("toy_latent", {"latent": self.latent}, {"q": f"{p}.lq", "c": f"{p}.lc", "out": f"{p}.lo"})
            layers.append(LayerSpec("prenorm", {
                "mixer": mixer, "mixer_norm": norm(f"{p}.n1"), "ffn_norm": norm(f"{p}.n2"),
                "ffn": PartSpec("swiglu", {"intermediate_size": self.intermediate_size},
                                {"gate": f"{p}.gate", "up": f"{p}.up", "down": f"{p}.down"})}))
        return ModelSpec(self.architecture, self.hidden_size, self.vocab_size, self.max_position_embeddings, layers,
                         [LayerCall(0), LayerCall(1), LayerCall(2)], norm("z.norm"),
                         PartSpec("embedding", {}, {"weight": "z.embed"}), PartSpec("lm_head", {"tied": False}, {"weight": "z.head"}))


register_architecture("ToyLatentForCausalLM", ToyLatentConfig)


def plain_latent_forward(cfg: ToyLatentConfig, W: Dict[str, torch.Tensor], tokens: List[int], stored=None) -> torch.Tensor:
    """Whole sequence, no cache, float64: the latent toy model written out plainly.  ``stored`` (for instance
    ``plain.as_bfloat16``) is applied to every value that a 16-bit engine keeps in 16 bits (normed rows, rotated
    queries and keys, values, attention's probabilities and output, the compressed vectors in their pages, gated
    activations): the distance of that run from the exact one is the noise of the storage type."""
    import plain
    keep = stored if stored is not None else (lambda t: t)
    W = {k: v.double() for k, v in W.items()}
    T = len(tokens)
    H, KV, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    h = W["z.embed"][torch.tensor(tokens)]
    inv = plain.rope_inv_freq(D, 1e4, None)
    pos = torch.arange(T)
    for l in range(3):
        p = f"z.{l}"
        x = keep(plain.rmsnorm(h, W[f"{p}.n1"], 1e-5))
        if l == 1:
            q = keep(plain.rope((x @ W[f"{p}.q"].T).reshape(T, H, D), pos, inv))
            k = keep(plain.rope((x @ W[f"{p}.k"].T).reshape(T, KV, D), pos, inv))
            v = keep((x @ W[f"{p}.v"].T).reshape(T, KV, D))
            h = h + keep(plain.attention(q, k, v, D ** -0.5, stored=stored)) @ W[f"{p}.o"].T
        else:
            q, c = x @ W[f"{p}.lq"].T, keep(x @ W[f"{p}.lc"].T)
            ys = []
            for t in range(T):
                pr = torch.softmax(c[: t + 1] @ q[t] / cfg.latent ** 0.5, dim=0)
                ys.append((pr @ c[: t + 1]) @ W[f"{p}.lo"].T)
            h = h + torch.stack(ys)
        x = keep(plain.rmsnorm(h, W[f"{p}.n2"], 1e-5))
        h = h + plain.swiglu_ffn(x, W[f"{p}.gate"], W[f"{p}.up"], W[f"{p}.down"], stored)
    return keep(plain.rmsnorm(h, W["z.norm"], 1e-5)) @ W["z.head"].T
