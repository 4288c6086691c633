"""Gedatar: a hybrid decoder-only stack whose layers each name their own token mixer.

Per layer (x is the fp32 residual stream, DyT(z) = tanh(alpha z) * w + b with a scalar alpha):

    h  = DyT_1(x);  h <- h + causal depthwise conv over time (``canon_taps`` taps, no bias)
    x <- x + DyT_1b(mixer(h))
    x <- x + DyT_2b(ff(DyT_2(x)))            (layers without a feed-forward skip this line)

Mixers: ``attention`` (grouped-query, values are the un-normalised keys, q / k unit-RMS per head,
no rotation, block-diagonal causal mask of ``mask.size`` positions, softmax with a zero-score
sink), ``wkv`` (RWKV-style token shift + per-channel decay + current-token bonus) and
``general_delta`` (decay + rank-one removal along the unit key + rank-one write).
Feed-forwards: SwiGLU, dense or a top-k mixture of experts with a shared expert.

The checkpoint names tensors ``l<i>.<part>`` / ``embed`` / ``final.norm`` / ``head``; this module
keeps exactly those names (``model.tensor(name)``), so loading is a strict name-and-shape match.
The serving path (``lumen.serve.hybrid_runner``) reads the tensors from here and runs the HIP
kernels of ``lumen/csrc/seqmix``; ``forward`` below is the same step function on fresh state.
"""
from __future__ import annotations

import math
from typing import Dict, Tuple

import torch

from .config import ModelConfig
from .named import NamedTensorModel

MIXERS = ("attention", "wkv", "general_delta")
# general_delta's decay is exp(-DELTA_DECAY * sigmoid(.)): the design fixes the constant
DELTA_DECAY = math.exp(-0.5)
# general_delta normalises its key by sqrt(sum k^2 + DELTA_KEY_EPS)
DELTA_KEY_EPS = 1e-6
DEFAULT_DECAY_RANK = 16


def _norm(out: Dict[str, tuple], name: str, W: int):
    out[name] = (W,)
    out[name + ".b"] = (W,)
    out[name + ".alpha"] = ()


def _ffn(out, p, W, ff):
    out[p + "gate"] = (ff, W)
    out[p + "up"] = (ff, W)
    out[p + "down"] = (W, ff)


def tensor_shapes(cfg: ModelConfig, decay_rank: int = DEFAULT_DECAY_RANK) -> Dict[str, tuple]:
    """{checkpoint tensor name: shape} of a configuration.  The decay projections' inner size is
    not part of the configuration (a checkpoint's ``w1`` shape gives it)."""
    W, V = cfg.hidden_size, cfg.vocab_size
    out: Dict[str, tuple] = {"embed": (V, W)}
    for i, L in enumerate(cfg.layer_specs):
        p = f"l{i}."
        m = L["mixer"]
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if L.get("mlp") else ()):
            _norm(out, p + n, W)
        out[p + "canon1"] = (W, cfg.canon_taps)
        x = p + "mix."
        if L["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m.get("vdim", m["dim"])
            out[x + "q"] = (H * D, W)
            out[x + "k"] = (G * D, W)
            out[x + "o"] = (W, H * Dv)
        else:
            HD = m["heads"] * m["dim"]
            for n in ("r", "k", "v", "g"):
                out[x + n] = (HD, W)
            out[x + "w1"] = (decay_rank, W)
            out[x + "w2"] = (HD, decay_rank)
            out[x + "w0"] = (HD,)
            out[x + "norm"] = (HD,)
            out[x + "o"] = (W, HD)
            if L["type"] == "wkv":
                for n in "rkvgw":
                    out[x + "mu." + n] = (W,)
                out[x + "u"] = (m["heads"], m["dim"])
            else:
                out[x + "a"] = (HD, W)
                out[x + "a.b"] = (HD,)
        f = L.get("mlp")
        if f:
            y = p + "mlp."
            if f["kind"] == "dense":
                _ffn(out, y, W, f["ff"])
            else:
                E = f["router"]["experts"]
                for e in range(E):
                    _ffn(out, y + f"e{e}.", W, f["expert"]["ff"])
                out[y + "router"] = (E, W)
                out[y + "router.b"] = (E,)
                if f.get("shared"):
                    _ffn(out, y + "shared.", W, f["shared"]["ff"])
    _norm(out, "final.norm", W)
    out["head"] = (V, W)
    return out


def validate(cfg: ModelConfig) -> None:
    """Reject configurations the kernels cannot run, with the reason."""
    for i, L in enumerate(cfg.layer_specs):
        m = L["mixer"]
        if L["type"] == "attention":
            if m["heads"] % m["kv_heads"]:
                raise ValueError(f"layer {i}: heads {m['heads']} not a multiple of kv_heads "
                                 f"{m['kv_heads']}")
            if m.get("vdim", m["dim"]) != m["dim"]:
                raise ValueError(f"layer {i}: the values are the keys, so vdim must equal dim")
            if int(m["mask"]["size"]) < 1:
                raise ValueError(f"layer {i}: mask.size must be >= 1")
            if m["dim"] > 256:
                raise ValueError(f"layer {i}: attention head size {m['dim']} > 256 is not "
                                 "supported")
        elif m["dim"] > 256:
            raise ValueError(f"layer {i}: recurrent head size {m['dim']} > 256 is not supported")
        f = L.get("mlp")
        if f and f["kind"] == "moe" and not 1 <= f["router"]["top"] <= f["router"]["experts"]:
            raise ValueError(f"layer {i}: top must be in [1, experts]")
    if not 1 <= cfg.canon_taps <= 16:
        raise ValueError(f"canon.taps must be in [1, 16], got {cfg.canon_taps}")


class GedatarForCausalLM(NamedTensorModel):
    supports_packing = False

    def __init__(self, config: ModelConfig, dtype=torch.bfloat16, device=None,
                 decay_rank: int = DEFAULT_DECAY_RANK):
        validate(config)
        super().__init__(config, tensor_shapes(config, decay_rank), dtype, device)

    @torch.no_grad()
    def init_weights(self, std: float = 0.02, seed: int = 0):
        """Random weights for synthetic runs: projections Normal(0, 1 / sqrt(fan_in)), norm
        weights near 1, decay offsets spread so that fast and slow channels both occur."""
        g = torch.Generator(device="cpu").manual_seed(seed)
        for name in self.tensor_names():
            p = self.tensor(name)
            leaf = name.rsplit(".", 1)[-1]
            if p.dim() == 0:                                   # DyT alpha
                v = torch.full((), 0.5) + 0.5 * torch.rand((), generator=g)
            elif p.dim() == 2 and leaf not in ("canon1", "u"):
                v = torch.randn(p.shape, generator=g) / math.sqrt(p.shape[1])
            elif leaf == "canon1":
                v = 0.3 * torch.randn(p.shape, generator=g)
            elif leaf == "u":
                v = 0.5 * torch.randn(p.shape, generator=g)
            elif leaf == "w0":
                v = torch.linspace(-3.0, 1.0, p.numel())[torch.randperm(p.numel(), generator=g)]
            elif leaf == "b" and ".norm" not in name and "final" not in name:
                v = 0.1 * torch.randn(p.shape, generator=g)    # router / removal-rate bias
            elif leaf == "b":
                v = 0.05 * torch.randn(p.shape, generator=g)   # DyT shift
            elif leaf in "rkvgw" and ".mu." in name:
                v = torch.rand(p.shape, generator=g)
            else:                                              # norm weights
                v = 1.0 + 0.1 * torch.randn(p.shape, generator=g)
            p.copy_(v.to(p.dtype))

    # ---- whole sequences on fresh state ----------------------------------------------------
    @torch.no_grad()
    def forward(self, input_ids: torch.Tensor) -> torch.Tensor:
        """Logits [B, S, V] of whole sequences starting at position 0: the serving step function
        (``lumen.serve.hybrid_runner``) on a private cache, every row's logits kept."""
        from ..serve.hybrid_runner import forward_fresh

        if input_ids.dim() == 1:
            input_ids = input_ids.view(1, -1)
        return forward_fresh(self, input_ids)


@torch.no_grad()
def load_gedatar_weights(model: GedatarForCausalLM, handles: dict, path: str) -> None:
    """Strict load: every tensor the configuration implies must be in the checkpoint with its
    shape, and the checkpoint may hold nothing else.  Only the decay projections' inner size is
    taken from the file."""
    names = set(model.tensor_names())
    extra = sorted(set(handles) - names)
    missing = sorted(names - set(handles))
    if missing or extra:
        raise KeyError(f"{path}: missing tensors {missing[:6]}, unexpected tensors {extra[:6]}")
    for name in model.tensor_names():
        t = handles[name].get_tensor(name)
        dst = model.tensor(name)
        if tuple(t.shape) != tuple(dst.shape):
            leaf = name.rsplit(".", 1)[-1]
            rank_only = (leaf == "w1" and t.dim() == 2 and t.shape[1] == dst.shape[1]) or (
                leaf == "w2" and t.dim() == 2 and t.shape[0] == dst.shape[0])
            if not rank_only:
                raise ValueError(f"{name}: checkpoint {tuple(t.shape)} != model "
                                 f"{tuple(dst.shape)}")
            model.replace_tensor(name, torch.empty(t.shape, dtype=dst.dtype, device=dst.device))
            dst = model.tensor(name)
        if not t.is_floating_point():
            raise ValueError(f"{name}: expected a floating-point tensor, got {t.dtype}")
        dst.copy_(t.to(dst.dtype))
    for i, L in enumerate(model.config.layer_specs):
        if L["type"] != "attention":
            a, b = model.tensor(f"l{i}.mix.w1"), model.tensor(f"l{i}.mix.w2")
            if a.shape[0] != b.shape[1]:
                raise ValueError(f"l{i}.mix: w1 {tuple(a.shape)} and w2 {tuple(b.shape)} disagree")
