"""Dalavik: a decoder-only stack of latent-attention and grouped-query attention layers.

Per layer (x is the fp32 residual stream; the sublayers read x itself, the norm sits on their
OUTPUT; gnorm = RMS norm in ``norm_groups`` consecutive groups with a plain weight):

    x <- x + gnorm_1(mixer(x))
    x <- x + gnorm_2(W_down (relu(W_gate x) * (W_up x)))             (layers with a feed-forward)
    x <- x + rms(W_proj (gelu_tanh(W_sgate x) * E[token, i*d:(i+1)*d])) * w_side   (token side input)

Mixers:

``latent_attention``  queries through a normed latent (c_q = rms(W_dq x) * w, q = W_uq c_q, per
    head [dim plain | rot_dim rotated]); keys and values from ONE cached row per token, the
    normed latent c (kv_rank) and a rotated key part shared by all heads (rot_dim):
    score = (q_plain . W_uk c + q_rot . k_rot) * scale, value = W_uv c, plain causal softmax.
    Interleaved rotary (pairs (2i, 2i+1), angle p * base^(-2i / dims)).  A layer with
    ``kv_from: j`` has no down projection of its own: it reads layer j's cached rows with its own
    W_uk / W_uv.  The serving path never expands the cache: q_plain is projected into the latent
    space (W_uk^T q) and the value projection is applied to the attention-weighted latent.

``attention``  grouped-query attention with biased projections, per-head RMS norm of q and k
    (one weight each, shared by the heads), no rotation; the score is multiplied by a
    position-dependent query temperature 1 + coef * ln(floor((p + 1) / every) + 1), soft-capped
    (cap * tanh(s / cap)), lowered by a per-head distance bias r1 * ln(1 + r2 * (i - j)), mixed
    across the heads (s_h <- sum_g talk[h, g] s_g) and normalised by a softmax whose denominator
    also holds exp(sink_h).

Output: gnorm with ``final.norm``, logits through the (tied) embedding table.

The checkpoint names tensors ``embed`` / ``side.embed`` / ``l<i>.<part>`` / ``final.norm``; this
module keeps exactly those names.  The serving step function is
``lumen.serve.hybrid_runner.DalavikWeights.run_layers``; ``forward`` runs it on fresh caches.
"""
from __future__ import annotations

import math
from typing import Dict

import torch

from .config import ModelConfig
from .named import NamedTensorModel

MIXERS = ("latent_attention", "attention")


def tensor_shapes(cfg: ModelConfig) -> Dict[str, tuple]:
    """{checkpoint tensor name: shape} of a configuration."""
    W, V = cfg.hidden_size, cfg.vocab_size
    n_layers = len(cfg.layer_specs)
    out: Dict[str, tuple] = {"embed": (V, W)}
    sd = cfg.token_side_dim
    if sd:
        out["side.embed"] = (V, n_layers * sd)
    for i, L in enumerate(cfg.layer_specs):
        p, m = f"l{i}.", L["mixer"]
        x = p + "mix."
        out[p + "norm1"] = (W,)
        if L["type"] == "latent_attention":
            H, D, Dr, Dv, R, Q = (m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"],
                                  m["q_rank"])
            out[x + "dq"] = (Q, W)
            out[x + "dq.norm"] = (Q,)
            out[x + "uq"] = (H * (D + Dr), Q)
            if m.get("kv_from") is None:
                out[x + "dkv"] = (R + Dr, W)
                out[x + "dkv.norm"] = (R,)
            out[x + "uk"] = (H * D, R)
            out[x + "uv"] = (H * Dv, R)
            out[x + "o"] = (W, H * Dv)
        else:
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out[x + "q"], out[x + "q.b"] = (H * D, W), (H * D,)
            out[x + "k"], out[x + "k.b"] = (G * D, W), (G * D,)
            out[x + "v"], out[x + "v.b"] = (G * Dv, W), (G * Dv,)
            out[x + "q.norm"] = out[x + "k.norm"] = (D,)
            out[x + "r1"] = out[x + "r2"] = out[x + "sink"] = (H,)
            out[x + "talk"] = (H, H)
            out[x + "o"] = (W, H * Dv)
        f = L.get("mlp")
        if f:
            out[p + "norm2"] = (W,)
            out[p + "mlp.gate"] = out[p + "mlp.up"] = (f["ff"], W)
            out[p + "mlp.down"] = (W, f["ff"])
        if sd:
            out[p + "side.gate"] = (sd, W)
            out[p + "side.proj"] = (W, sd)
            out[p + "side.norm"] = (W,)
    out["final.norm"] = (W,)
    return out


def validate(cfg: ModelConfig) -> None:
    """Reject configurations the step function or its kernels cannot run, with the reason."""
    if cfg.norm_groups < 1 or cfg.hidden_size % cfg.norm_groups:
        raise ValueError(f"width {cfg.hidden_size} is not a multiple of norm.groups "
                         f"{cfg.norm_groups}")
    for i, L in enumerate(cfg.layer_specs):
        m = L["mixer"]
        if L["type"] == "latent_attention":
            rot = m["rot"]
            if rot["dims"] % 2 or rot["dims"] > m["rot_dim"]:
                raise ValueError(f"layer {i}: rot.dims {rot['dims']} must be even and at most "
                                 f"rot_dim {m['rot_dim']}")
            if m["kv_rank"] > 512:
                raise ValueError(f"layer {i}: kv_rank {m['kv_rank']} > 512 is not supported")
            j = m.get("kv_from")
            if j is not None:
                if not 0 <= j < i or cfg.layer_specs[j]["type"] != "latent_attention" or \
                        cfg.layer_specs[j]["mixer"].get("kv_from") is not None:
                    raise ValueError(f"layer {i}: kv_from {j} must name an earlier "
                                     "latent_attention layer with a cache of its own")
                o = cfg.layer_specs[j]["mixer"]
                if (o["kv_rank"], o["rot_dim"], o["rot"]) != (m["kv_rank"], m["rot_dim"], rot):
                    raise ValueError(f"layer {i}: kv_rank / rot_dim / rot differ from layer {j}'s")
        else:
            if m["heads"] % m["kv_heads"]:
                raise ValueError(f"layer {i}: heads {m['heads']} not a multiple of kv_heads "
                                 f"{m['kv_heads']}")
            if m["vdim"] > 512:
                raise ValueError(f"layer {i}: vdim {m['vdim']} > 512 is not supported")
            if m["heads"] > 32:
                raise ValueError(f"layer {i}: head mixing over {m['heads']} > 32 heads is not "
                                 "supported")
        f = L.get("mlp")
        if f and f.get("kind", "dense") != "dense":
            raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")


class DalavikForCausalLM(NamedTensorModel):
    supports_packing = False

    def __init__(self, config: ModelConfig, dtype=torch.bfloat16, device=None):
        validate(config)
        super().__init__(config, tensor_shapes(config), dtype, device)

    @torch.no_grad()
    def init_weights(self, std: float = 0.02, seed: int = 0):
        """Random weights for synthetic runs: projections Normal(0, 1 / sqrt(fan_in)), norm
        weights near 1, small biases, distance-bias rates positive, head mixing near identity."""
        g = torch.Generator(device="cpu").manual_seed(seed)
        for name in self.tensor_names():
            p = self.tensor(name)
            leaf = name.rsplit(".", 1)[-1]
            if leaf == "talk":
                v = torch.eye(p.shape[0]) + 0.2 * torch.randn(p.shape, generator=g)
            elif name.endswith("embed"):
                v = torch.randn(p.shape, generator=g)
            elif p.dim() == 2:
                v = torch.randn(p.shape, generator=g) / math.sqrt(p.shape[1])
            elif leaf == "b":
                v = 0.1 * torch.randn(p.shape, generator=g)
            elif leaf == "r1":
                v = 0.3 * torch.rand(p.shape, generator=g)
            elif leaf == "r2":
                v = 0.05 + 0.5 * torch.rand(p.shape, generator=g)
            elif leaf == "sink":
                v = torch.randn(p.shape, generator=g)
            else:                                              # norm weights
                v = 1.0 + 0.1 * torch.randn(p.shape, generator=g)
            p.copy_(v.to(p.dtype))

    @torch.no_grad()
    def forward(self, input_ids: torch.Tensor) -> torch.Tensor:
        """Logits [B, S, V] of whole sequences starting at position 0: the serving step function
        on a private cache, every row's logits kept."""
        from ..serve.hybrid_runner import forward_fresh

        if input_ids.dim() == 1:
            input_ids = input_ids.view(1, -1)
        return forward_fresh(self, input_ids)


@torch.no_grad()
def load_dalavik_weights(model: DalavikForCausalLM, handles: dict, path: str) -> None:
    """Every tensor the configuration implies must be in the checkpoint with its shape; tensors
    the configuration has no use for are listed in ``model.ignored_tensors`` and not read."""
    names = model.tensor_names()
    missing = sorted(set(names) - set(handles))
    if missing:
        raise KeyError(f"{path}: missing tensors {missing[:8]}")
    model.ignored_tensors = sorted(set(handles) - set(names))
    for name in names:
        t = handles[name].get_tensor(name)
        dst = model.tensor(name)
        if tuple(t.shape) != tuple(dst.shape):
            raise ValueError(f"{name}: checkpoint {tuple(t.shape)} != model {tuple(dst.shape)}")
        if not t.is_floating_point():
            raise ValueError(f"{name}: expected a floating-point tensor, got {t.dtype}")
        dst.copy_(t.to(dst.dtype))
