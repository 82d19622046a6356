"""A toy architecture defined entirely in the tests: a mixer with per-request state of its own (a decaying
running sum, no paged cache), used in some layers beside attention in others, registered through the public
registries.  Nothing under tempura_amd/ knows about it."""
from __future__ import annotations

import json
from dataclasses import dataclass
from typing import Dict, List

import torch

from tempura_amd.config import LayerCall, LayerSpec, ModelSpec, PartSpec, register_architecture
from tempura_amd.parts import Mixer, StateSpec, WeightInfo, register_part


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
                mixer = PartSpec("decay_sum", {"width": self.width, "decay": self.decay},
                                 {"in": f"{p}.mix.in", "out": f"{p}.mix.out"})
            else:
                mixer = PartSpec("attention", {"num_heads": self.num_attention_heads, "num_kv_heads": 2,
                                               "head_dim": self.head_dim, "scale": self.head_dim ** -0.5, "window": None,
                                               "position": PartSpec("rope", {"head_dim": self.head_dim, "theta": 1e4, "scaling": None})},
                                 {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o"})
            layers.append(LayerSpec(
                "prenorm", mixer,
                PartSpec("swiglu", {"intermediate_size": self.intermediate_size},
                         {"gate": f"{p}.gate", "up": f"{p}.up", "down": f"{p}.down"}),
                PartSpec("rmsnorm", {"eps": 1e-5}, {"weight": f"{p}.n1"}),
                PartSpec("rmsnorm", {"eps": 1e-5}, {"weight": f"{p}.n2"})))
        return ModelSpec(self.architecture, self.hidden_size, self.vocab_size, self.max_position_embeddings, layers,
                         [LayerCall(l) for l in range(self.num_hidden_layers)],
                         PartSpec("rmsnorm", {"eps": 1e-5}, {"weight": "toy.norm"}),
                         PartSpec("embedding", {}, {"weight": "toy.embed"}),
                         PartSpec("lm_head", {"tied": True, "tied_to": "toy.embed"}, {"weight": "toy.head"}))


register_architecture("ToyForCausalLM", ToyConfig)


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
