"""Parts and architectures that exist only in the tests.  They are registered
through the framework's public registries, without a change to its files, and
show what the interfaces carry: a mixer with per-request state of its own, a
run order that names a layer twice and lets an entry read another entry's cache,
and layers with a sliding window (a cache group of their own).  None of them is
a model of anyone's; the plain references sit beside them.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

import plain_llama
from tokasaurus_amd.config.model_config import LlamaConfig
from tokasaurus_amd.kernels import ops
from tokasaurus_amd.models import Architecture, ModelSpec, RunEntry, register_architecture
from tokasaurus_amd.models.llama import llama_spec
from tokasaurus_amd.parts.base import MIXERS, NORM_WEIGHT, Mixer, PartSpec, StateNeed, TensorSpec
from tokasaurus_amd.parts.linear import Linear

# --------------------------------------------------------------------------
# a mixer with state: s_t = a * s_{t-1} + W_in h_t,  y_t = W_out s_t
# --------------------------------------------------------------------------


@MIXERS.register("toy_recurrence", replace=True)
class ToyRecurrence(Mixer):
    """Keeps one vector of ``state_size`` 32-bit numbers per request, in the
    request's slot.  A request's state starts from zero at position 0."""

    def __init__(self, hidden_size: int, state_size: int, names: dict[str, str]):
        self.hidden_size, self.state_size = hidden_size, state_size
        self.inp = Linear(hidden_size, [names["in"]], [state_size])
        self.out = Linear(state_size, [names["out"]], [hidden_size])
        self.decay_name = names["decay"]
        self.decay: torch.Tensor | None = None

    def tensor_specs(self) -> list[TensorSpec]:
        return self.inp.tensor_specs() + self.out.tensor_specs() + [TensorSpec(self.decay_name, (self.state_size,), NORM_WEIGHT)]

    def state_need(self) -> StateNeed:
        return StateNeed((self.state_size,), torch.float32)

    def load(self, tensors, placer) -> None:
        self.inp.load(tensors, placer)
        self.out.load(tensors, placer)
        self.decay = placer.place(("vector", self.decay_name), lambda: (0.5 * tensors[self.decay_name].float()).to(placer.device))

    def forward(self, h, residual, ctx, cache, state, rows):
        assert cache is None and state is not None
        u = ops.gemm_generic(h, self.inp.weight, out_f32=True)  # [N, S] 32-bit
        if ctx.max_q_len == 1:
            # one token a request: device arrays only, so the step can be recorded and replayed
            slots = ctx.slots.long()
            prev = state.index_select(0, slots)
            prev = torch.where((ctx.positions == 0)[:, None], torch.zeros_like(prev), prev)
            s_all = self.decay[None, :] * prev + u
            state.index_copy_(0, slots, s_all)
        else:
            s_all = torch.empty_like(u)
            for r in range(ctx.num_requests):
                a, b = ctx.host_q_start[r], ctx.host_q_start[r + 1]
                start = ctx.host_kv_len[r] - (b - a)
                s = state[ctx.host_slots[r]].clone() if start > 0 else torch.zeros_like(state[0])
                for t in range(a, b):
                    s = self.decay * s + u[t]
                    s_all[t] = s
                state[ctx.host_slots[r]] = s
        y = ops.gemm_generic(s_all.to(h.dtype), self.out.weight)
        if rows is not None:
            y = ops.gather_rows(y, rows)
        return ops.add(y, residual.contiguous())


def plain_recurrence(h: torch.Tensor, w: dict, prefix: str) -> torch.Tensor:
    """The toy mixer on one whole sequence: h [T, H] -> y [T, H]."""
    a = 0.5 * w[f"{prefix}.mixer.decay"]
    s = torch.zeros_like(a)
    out = []
    for t in range(h.shape[0]):
        s = a * s + w[f"{prefix}.mixer.in.weight"] @ h[t]
        out.append(w[f"{prefix}.mixer.out.weight"] @ s)
    return torch.stack(out)


@dataclass(frozen=True)
class ToyConfig:
    llama: LlamaConfig
    state_size: int
    recurrent_layers: tuple[int, ...]

    @staticmethod
    def from_dict(d: dict[str, Any]) -> "ToyConfig":
        return ToyConfig(LlamaConfig.from_dict(d), int(d["toy_state_size"]), tuple(d["toy_recurrent_layers"]))


def toy_recurrent_spec(cfg: ToyConfig) -> ModelSpec:
    base = llama_spec(cfg.llama)
    layers = list(base.layers)
    for i in cfg.recurrent_layers:
        p = f"model.layers.{i}"
        params = dict(layers[i].params)
        params["mixer"] = PartSpec(
            "toy_recurrence",
            {"hidden_size": cfg.llama.hidden_size, "state_size": cfg.state_size,
             "names": {"in": f"{p}.mixer.in.weight", "out": f"{p}.mixer.out.weight", "decay": f"{p}.mixer.decay"}},
        )
        layers[i] = PartSpec(layers[i].kind, params)
    return ModelSpec(**{**base.__dict__, "layers": tuple(layers)})


def plain_toy_recurrent_logits(cfg: dict, w: dict, token_ids: list[int]) -> torch.Tensor:
    d = cfg["hidden_size"] // cfg["num_attention_heads"]
    x = w["model.embed_tokens.weight"][torch.tensor(token_ids)]
    inv = plain_llama.rope_inverse_frequencies(d, float(cfg["rope_theta"]), cfg.get("rope_scaling"))
    cos, sin = plain_llama.rope_tables(torch.arange(len(token_ids)), inv)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        if i in cfg["toy_recurrent_layers"]:
            h = plain_llama.rms_norm(x, w[f"{p}.input_layernorm.weight"], cfg["rms_norm_eps"])
            x = x + plain_recurrence(h, w, p)
        else:
            x = plain_llama.attention_block(x, w, p, cfg, cos, sin)
        x = plain_llama.swiglu_block(x, w, p, cfg)
    return plain_llama.lm_head(x, w, cfg)


# --------------------------------------------------------------------------
# Llama's parts in another arrangement: a run order as data, windows per layer
# --------------------------------------------------------------------------


@dataclass(frozen=True)
class ArrangedConfig:
    llama: LlamaConfig
    run_order: tuple[tuple[int, int | None], ...]  # (layer, place whose cache is read or None)
    windows: dict[int, int]

    @staticmethod
    def from_dict(d: dict[str, Any]) -> "ArrangedConfig":
        order = tuple((int(e[0]), None if e[1] is None else int(e[1])) for e in d["toy_run_order"])
        return ArrangedConfig(LlamaConfig.from_dict(d), order, {int(k): int(v) for k, v in d.get("toy_windows", {}).items()})


def arranged_spec(cfg: ArrangedConfig) -> ModelSpec:
    base = llama_spec(cfg.llama)
    layers = list(base.layers)
    for i, window in cfg.windows.items():
        params = dict(layers[i].params)
        mixer = params["mixer"]
        params["mixer"] = PartSpec(mixer.kind, {**mixer.params, "window": window})
        layers[i] = PartSpec(layers[i].kind, params)
    order = tuple(RunEntry(layer, cache_of) for layer, cache_of in cfg.run_order)
    return ModelSpec(**{**base.__dict__, "layers": tuple(layers), "run_order": order})


def plain_arranged_logits(cfg: dict, w: dict, token_ids: list[int]) -> torch.Tensor:
    order = [e[0] for e in cfg["toy_run_order"]]
    kv_from = {place: e[1] for place, e in enumerate(cfg["toy_run_order"]) if e[1] is not None}
    windows = {int(k): int(v) for k, v in cfg.get("toy_windows", {}).items()}
    return plain_llama.forward_logits(cfg, w, token_ids, layer_order=order, windows=windows, kv_from=kv_from)


def register() -> None:
    register_architecture(Architecture("toy_recurrent", ToyConfig.from_dict, toy_recurrent_spec), replace=True)
    register_architecture(Architecture("toy_arranged", ArrangedConfig.from_dict, arranged_spec), replace=True)
