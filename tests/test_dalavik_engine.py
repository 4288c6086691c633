"""Dalavik through the serving engine (model registry, loader, block manager, scheduler, hybrid
runner, trace replay) against the float64 whole-sequence oracle of tests/_ref_dalavik.py.

Every test runs on the CPU (the ops' torch path) and, marked ``gpu``, on the HIP kernels.  The
configurations are small and unlike each other: latent layers with their own and with a borrowed
cache, rotary on all and on a part of the rotated slice, head counts that are no multiple of the
kernel's waves, key / value / latent sizes that are and are not multiples of the vector width,
grouped, multi-query and full-head attention, with and without temperature and soft cap, one to
five norm groups, with and without the token side input, layers without a feed-forward."""
import os

import pytest
import torch

import _ref_dalavik as ref

from lumen.models import build_model
from lumen.models.config import ModelConfig, dalavik_to_dict, get_config
from lumen.models.dalavik import DalavikForCausalLM
from lumen.serve.engine import EngineConfig, LLMEngine
from lumen.serve.sequence import SamplingParams
from lumen.serve.trace import TraceReplay

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def _cfg(name, vocab, width, groups, side, eps, layers):
    return ModelConfig(arch="dalavik", vocab_size=vocab, hidden_size=width,
                       num_hidden_layers=len(layers), rms_norm_eps=eps, norm_groups=groups,
                       token_side_dim=side, intermediate_size=0, num_attention_heads=0,
                       num_key_value_heads=0, max_position_embeddings=1 << 20, eos_token_id=-1,
                       tie_word_embeddings=True, name=name, layer_specs=layers)


def _lat(H, D, Dr, Dv, R, Q, scale, base, dims, mlp, kv_from=None):
    m = {"heads": H, "dim": D, "rot_dim": Dr, "vdim": Dv, "kv_rank": R, "q_rank": Q,
         "scale": scale, "rot": {"base": base, "dims": dims}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def _att(H, G, D, Dv, scale, mlp, softcap=None, q_temp=None):
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "scale": scale}
    if softcap:
        m["softcap"] = softcap
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def _ff(n):
    return {"kind": "dense", "ff": n}


CONFIGS = {
    "tiny": lambda: get_config("tiny-dalavik"),
    # nothing a multiple of 8: scalar key and value paths; 7 and 3 heads; rotary on a part of the
    # rotated slice; two borrowers of one cache, the lender first; no side input; five norm groups
    "odd": lambda: _cfg("odd", 131, 80, 5, 0, 3e-6, [
        _lat(7, 12, 6, 20, 22, 20, 0.21, 777.0, 4, _ff(56)),
        _att(3, 3, 20, 12, 0.3, None),
        _lat(2, 10, 6, 14, 22, 28, 0.3, 777.0, 4, None, kv_from=0),
        _lat(4, 18, 6, 6, 22, 12, 0.12, 777.0, 4, _ff(72), kv_from=0)]),
    # one of everything: one head, one key/value head, one norm group, temperature stepping at
    # every position, a latent wider than the heads it feeds
    "one": lambda: _cfg("one", 64, 48, 1, 5, 1e-4, [
        _att(1, 1, 16, 8, 0.4, _ff(40), softcap=3.0, q_temp=(0.7, 1)),
        _lat(1, 8, 4, 16, 40, 8, 0.25, 50.0, 4, _ff(24)),
        _att(8, 1, 8, 8, 0.35, None, q_temp=(0.05, 16))]),
    # latents of 128 and cache blocks of 16: in 16 bits the value product of the latent layers
    # runs on the matrix cores from the transposed copy; 18 heads make two head blocks
    "wide": lambda: _cfg("wide", 200, 128, 2, 0, 1e-5, [
        _lat(5, 32, 32, 24, 128, 48, 0.12, 10000.0, 32, _ff(96)),
        _att(4, 2, 32, 32, 0.2, None, softcap=8.0),
        _lat(18, 16, 32, 16, 128, 32, 0.15, 10000.0, 32, _ff(64), kv_from=0)]),
}


def make(name, device, dtype=torch.float32, seed=0):
    m = DalavikForCausalLM(CONFIGS[name](), dtype=dtype, device=device)
    m.init_weights(seed=seed)
    return m


class Oracle:
    def __init__(self, model):
        self.cfg = dalavik_to_dict(model.config)
        self.w = {n: model.tensor(n).detach().cpu() for n in model.tensor_names()}

    def forward(self, toks):
        return ref.forward(self.cfg, self.w, toks)


oracle = Oracle


class _NoTokenizer:
    eos_token_id = None


def engine(model, device, blocks=64, bs=16, seqs=4, budget=4096, graphs=True, **kw):
    return LLMEngine(EngineConfig(model=model.config.name, device=device, dtype="fp32" if
                                  model.dtype == torch.float32 else "bf16", num_blocks=blocks,
                                  block_size=bs, max_num_seqs=seqs, max_num_batched_tokens=budget,
                                  max_model_len=blocks * bs, use_graphs=graphs, **kw),
                     model=model, tokenizer=_NoTokenizer())


def tokens(model, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, model.config.vocab_size, (n,), generator=g).tolist()


def check(got, want, rtol=2e-4):
    got, want = got.to(ref.F64), want.to(ref.F64)
    scale = float(want.std())
    err = float((got - want).abs().max())
    assert err <= rtol * max(scale, 1.0), f"max error {err:.3e} at logit scale {scale:.3f}"


def replay_alone(model, device, toks, pieces, **kw):
    """One request fed in ``pieces`` (cycled); logits of every position."""
    rp = TraceReplay(engine(model, device, **kw))
    out, at, k = [], 0, 0
    while at < len(toks):
        c = min(pieces[k % len(pieces)], len(toks) - at)
        k += 1
        out.append(rp.step([{"id": "a", "tokens": toks[at:at + c], "want": list(range(c))}],
                           ["a"] if at + c == len(toks) else []))
        at += c
    return torch.cat(out, 0)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_matches_oracle(device, name):
    m = make(name, device)
    toks = tokens(m, 75, 1)
    want = oracle(m).forward(toks)
    check(replay_alone(m, device, toks, [1000]), want)
    # the model's own forward (fresh caches, every row) is the same step function
    check(m(torch.tensor(toks, device=device))[0].cpu(), want)


@pytest.mark.parametrize("device", DEVICES)
def test_residual_stream_after_every_layer(device):
    """The runner's per-layer hook against the oracle's stream: a fault shows at its layer."""
    m = make("tiny", device, seed=13)
    toks = tokens(m, 29, 14)
    layers = []
    o = oracle(m)
    ref.forward(o.cfg, o.w, toks, layers)
    eng = engine(m, device)
    seen = {}
    eng.runner.observe = lambda i, x: seen.__setitem__(i, x.detach().float().cpu().clone())
    TraceReplay(eng).step([{"id": "a", "tokens": toks, "want": []}], ["a"])
    assert sorted(seen) == list(range(len(layers)))
    for i, want in enumerate(layers):
        err = float((seen[i].to(ref.F64) - want).abs().max())
        assert err <= 1e-4 * max(1.0, float(want.abs().max())), f"layer {i}: {err:.3e}"


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_prefill_then_long_decode(device, name):
    """A short prompt, then token by token across several block borders and temperature steps."""
    m = make(name, device, seed=1)
    toks = tokens(m, 90, 2)
    want = oracle(m).forward(toks)
    check(replay_alone(m, device, toks, [5] + [1] * 200), want)
    # from the very first token on, one at a time (the first token is a one-row prefill)
    check(replay_alone(m, device, toks[:40], [1]), want[:40])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("pieces", [[2], [3, 1, 2, 17, 2, 1, 1, 30], [16], [15, 1, 17]])
def test_portions_of_several_sizes(device, pieces):
    m = make("tiny", device, seed=2)
    toks = tokens(m, 83, 3)
    check(replay_alone(m, device, toks, pieces, bs=8), oracle(m).forward(toks))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["tiny", "odd"])
def test_first_tokens(device, name):
    m = make(name, device, seed=3)
    orc = oracle(m)
    for n in (1, 2, 3):
        toks = tokens(m, n, 10 + n)
        check(replay_alone(m, device, toks, [1000]), orc.forward(toks))
        check(replay_alone(m, device, toks, [1]), orc.forward(toks))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["tiny", "odd"])
def test_mixed_batches_reuse_blocks(device, name):
    """Seven unequal requests through three sequence slots and a pool of 20 blocks of 8: portions
    of some beside single tokens of others; finished requests hand their blocks to new ones.
    Every request must come out as if it had run alone."""
    m = make(name, device, seed=4)
    orc = oracle(m)
    lens = [41, 9, 66, 2, 30, 17, 50]
    reqs = {f"r{i}": tokens(m, n, 20 + i) for i, n in enumerate(lens)}
    eng = engine(m, device, blocks=20, bs=8, seqs=3)
    rp = TraceReplay(eng)
    g = torch.Generator().manual_seed(5)
    waiting = list(reqs)
    live, at, got = [], {}, {r: [] for r in reqs}
    sizes = [2, 1, 1, 13, 1, 5, 1, 1, 24, 3]
    k = 0
    seen_blocks = []
    while waiting or live:
        while waiting and len(live) < 3:
            need = sum((len(reqs[r]) + 7) // 8 for r in live + [waiting[0]])
            if need > 20:
                break
            r = waiting.pop(0)
            live.append(r)
            at[r] = 0
        entries, end = [], []
        for r in list(live):
            if len(live) > 1 and torch.rand((), generator=g) < 0.3:
                continue                                   # left out of this step
            c = min(sizes[k % len(sizes)], len(reqs[r]) - at[r])
            k += 1
            entries.append({"id": r, "tokens": reqs[r][at[r]:at[r] + c], "want": list(range(c))})
            at[r] += c
            if at[r] == len(reqs[r]):
                end.append(r)
                live.remove(r)
        if not entries:
            continue
        out = rp.step(entries, end)
        seen_blocks += [b for t in eng.blocks.tables.values() for b in t]
        o = 0
        for e in entries:
            got[e["id"]].append(out[o:o + len(e["tokens"])])
            o += len(e["tokens"])
    assert eng.blocks.num_free == 20 and len(set(seen_blocks)) <= 20
    for r, toks in reqs.items():
        check(torch.cat(got[r], 0), orc.forward(toks))


@pytest.mark.parametrize("device", DEVICES)
def test_blocks_reused_after_finish(device):
    """The second request gets the first one's blocks (stale latents, keys and values)."""
    m = make("tiny", device, seed=6)
    orc = oracle(m)
    eng = engine(m, device, blocks=8, bs=16, seqs=1)
    rp = TraceReplay(eng)
    a, b = tokens(m, 100, 30), tokens(m, 60, 31)
    rp.step([{"id": "a", "tokens": a, "want": []}], ["a"])
    got = torch.cat([rp.step([{"id": "b", "tokens": b[:33], "want": list(range(33))}], []),
                     rp.step([{"id": "b", "tokens": b[33:], "want": list(range(27))}], ["b"])], 0)
    check(got, orc.forward(b))


@pytest.mark.parametrize("device", DEVICES)
def test_far_token_decides_through_both_mixers(device):
    """Weights made so that a fault in a far key shows: the query projections are scaled up, so
    the scores are sharp and a few keys -- wherever they lie -- carry a row's weight, and the
    distance bias is scaled down so that it cannot drown keys hundreds of positions back.  The
    prompt is fed whole, in ragged portions across block borders, and decoded token by token."""
    m = make("tiny", device, seed=21)
    with torch.no_grad():
        for i, L in enumerate(m.config.layer_specs):
            n = "q" if L["type"] == "attention" else "uq"
            m.tensor(f"l{i}.mix.{n}").mul_(6.0)            # sharp scores: few keys carry the weight
            if L["type"] == "attention":
                m.tensor(f"l{i}.mix.r1").mul_(0.05)        # and distance may not drown them
    toks = tokens(m, 260, 22)
    want = oracle(m).forward(toks)
    check(replay_alone(m, device, toks, [1000]), want, rtol=5e-4)
    check(replay_alone(m, device, toks, [37, 2, 50, 1, 64, 3], bs=8), want, rtol=5e-4)
    check(replay_alone(m, device, toks, [200] + [1] * 100), want, rtol=5e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["tiny", "one"])
def test_greedy_generation_through_scheduler(device, name):
    """LLMEngine.generate: chunked prefill under a small token budget, more prompts than
    sequence slots, async scheduling, greedy sampling -- every generated token is the oracle's
    arg-max (up to a tie within the tolerance) given the tokens before it."""
    m = make(name, device, seed=7)
    orc = oracle(m)
    eng = engine(m, device, blocks=48, bs=8, seqs=3, budget=24)
    prompts = [tokens(m, n, 40 + n) for n in (5, 37, 1, 20, 52)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True))
    assert eng.blocks.num_free == 48
    for p, s in zip(prompts, seqs):
        assert len(s.output_ids) == 10
        want = orc.forward(p + s.output_ids[:-1])
        for j, tok in enumerate(s.output_ids):
            row = want[len(p) - 1 + j]
            assert float(row.max() - row[tok]) <= 1e-3 * max(float(row.std()), 1.0)


@pytest.mark.parametrize("device", DEVICES)
def test_preemption_recomputes_caches(device):
    """A pool too small for all running sequences: the scheduler preempts and later recomputes a
    sequence from its first token in whatever blocks it then gets; outputs stay the oracle's."""
    m = make("odd", device, seed=8)
    orc = oracle(m)
    eng = engine(m, device, blocks=12, bs=4, seqs=3, budget=64, async_scheduling=False)
    prompts = [tokens(m, n, 60 + n) for n in (9, 11, 10)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=14, temperature=0.0, ignore_eos=True))
    assert eng.scheduler.num_preemptions > 0
    for p, s in zip(prompts, seqs):
        want = orc.forward(p + s.output_ids[:-1])
        for j, tok in enumerate(s.output_ids):
            row = want[len(p) - 1 + j]
            assert float(row.max() - row[tok]) <= 1e-3 * max(float(row.std()), 1.0)


def _random_config(seed):
    """A random stack: 2 - 5 layers of either mixer in any order, borrowers of earlier caches,
    sizes that are and are not multiples of the vector and matrix-core widths."""
    import random

    rng = random.Random(seed)
    W = rng.choice([64, 96, 160, 192])
    groups = rng.choice([g for g in (1, 2, 3, 4, 5, 8) if W % g == 0])
    layers, lenders = [], []
    for i in range(rng.randint(2, 5)):
        mlp = _ff(rng.choice([32, 48, 100])) if rng.random() < 0.8 else None
        if rng.random() < 0.6:
            if lenders and rng.random() < 0.4:
                src = rng.choice(lenders)
                o = layers[src]["mixer"]
                R, Dr, rot = o["kv_rank"], o["rot_dim"], o["rot"]
            else:
                src = None
                R, Dr = rng.choice([16, 24, 64, 72, 128]), rng.choice([4, 6, 8, 16, 32])
                rot = {"base": rng.choice([100.0, 10000.0, 500000.0]),
                       "dims": Dr if rng.random() < 0.7 else max(2, Dr // 4 * 2)}
            layers.append(_lat(rng.choice([1, 2, 3, 5, 8, 16, 17]), rng.choice([8, 12, 16, 40, 64]), Dr,
                               rng.choice([8, 16, 20, 32]), R, rng.choice([16, 24, 48]),
                               rng.uniform(0.05, 0.3), rot["base"], rot["dims"], mlp, src))
            if src is None:
                lenders.append(i)
        else:
            H = rng.choice([1, 2, 3, 4, 6, 8, 12, 32])
            G = rng.choice([g for g in (1, 2, 3, 4, H) if H % g == 0])
            layers.append(_att(H, G, rng.choice([8, 16, 20, 32, 64]), rng.choice([8, 12, 16, 48]),
                               rng.uniform(0.05, 0.3), mlp, softcap=rng.choice([None, 5.0, 30.0]),
                               q_temp=rng.choice([None, (0.3, 1), (0.2, 16), (0.1, 64)])))
    return _cfg(f"random{seed}", rng.randint(50, 400), W, groups, rng.choice([0, 4, 12, 16]),
                rng.choice([1e-6, 1e-5]), layers)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_configurations(device, seed):
    """Whole, in ragged portions, and decoded across a 128-key border: the oracle's logits (fp32)
    and, on the GPU in 16 bits, the same logits however the prompt was cut."""
    cfg = _random_config(seed)
    m = DalavikForCausalLM(cfg, dtype=torch.float32, device=device)
    m.init_weights(seed=seed)
    toks = tokens(m, 150, seed)
    want = oracle(m).forward(toks)
    for pieces in ([1000], [37, 2, 1, 50, 1, 1, 1, 3], [120] + [1] * 30):
        check(replay_alone(m, device, toks, pieces), want, rtol=5e-4)
    if device == "cuda":
        m16 = DalavikForCausalLM(cfg, dtype=torch.bfloat16, device=device)
        m16.init_weights(seed=seed)
        whole = replay_alone(m16, device, toks, [1000])
        check_rounding(replay_alone(m16, device, toks, [37, 2, 1, 50, 1, 1, 1, 3]), whole, rms=1e-2,
                       worst=0.25)
        check_rounding(replay_alone(m16, device, toks, [120] + [1] * 30), whole, rms=1e-2, worst=0.25)


def test_configuration_is_validated():
    bad = CONFIGS["odd"]()
    bad.layer_specs[2]["mixer"]["kv_from"] = 3            # a later layer cannot lend its cache
    with pytest.raises(ValueError):
        DalavikForCausalLM(bad, dtype=torch.float32, device="cpu")
    bad = CONFIGS["odd"]()
    bad.layer_specs[3]["mixer"]["kv_rank"] = 16           # a borrower must match the lender
    with pytest.raises(ValueError):
        DalavikForCausalLM(bad, dtype=torch.float32, device="cpu")
    bad = CONFIGS["tiny"]()
    bad.norm_groups = 7
    with pytest.raises(ValueError):
        DalavikForCausalLM(bad, dtype=torch.float32, device="cpu")


def test_checkpoint_roundtrip(tmp_path):
    """save -> config.json + model.safetensors under the design's tensor names -> load by
    directory (the class is picked by config.json); a missing tensor or a wrong shape is an
    error."""
    from safetensors.torch import load_file, save_file

    from lumen.models.loading import save_hf_weights

    for name in ("tiny", "odd"):
        m = make(name, "cpu", dtype=torch.bfloat16)
        d = str(tmp_path / name)
        save_hf_weights(m, d)
        m2 = build_model(d, dtype=torch.bfloat16, device="cpu")
        assert m2.config.arch == "dalavik" and type(m2) is DalavikForCausalLM
        assert m2.config.norm_groups == m.config.norm_groups
        assert m2.config.token_side_dim == m.config.token_side_dim
        for n in m.tensor_names():
            assert torch.equal(m.tensor(n), m2.tensor(n)), n
    f = os.path.join(d, "model.safetensors")
    sd = load_file(f)
    short = dict(sd)
    short.pop("l2.mix.uk")
    save_file(short, f)
    with pytest.raises(KeyError):
        build_model(d, dtype=torch.bfloat16, device="cpu")
    sd["l1.mix.r1"] = torch.zeros(5, dtype=torch.bfloat16)
    save_file(sd, f)
    with pytest.raises(ValueError):
        build_model(d, dtype=torch.bfloat16, device="cpu")


def test_trace_run_command_line(tmp_path):
    """bin/trace_run as a user runs it: a checkpoint directory, JSON steps on stdin, one logits
    file per step that wants any, `done <step>` after every step, exit code 0 at end of input."""
    import json
    import subprocess
    import sys

    import numpy as np

    from lumen.models.loading import save_hf_weights

    m = make("odd", "cpu", dtype=torch.bfloat16)
    d = str(tmp_path / "ckpt")
    out = str(tmp_path / "out")
    save_hf_weights(m, d)
    a, b = tokens(m, 21, 70), tokens(m, 12, 71)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:9], "want": [0, 8]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[9:10], "want": []},
                                     {"id": "b", "tokens": b[:11], "want": [10]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[11:], "want": [0]},
                                     {"id": "a", "tokens": a[10:], "want": [10]}],
              "end": ["a", "b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d,
                        "--dtype", "float32", "--out", out, "--max-tokens", "128", "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                       text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    orc = oracle(m)
    ra, rb = orc.forward(a), orc.forward(b)
    V = m.config.vocab_size
    got = {i: torch.from_numpy(np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4")).view(-1, V)
           for i in range(3)}
    check(got[0], ra[[0, 8]])
    check(got[1], rb[[10]])
    check(got[2], torch.stack([rb[11], ra[20]]))


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["tiny", "odd", "wide"])
def test_bf16_close_to_oracle_and_cut_invariant(name):
    """bf16 serving: within rounding of the float64 oracle, and the same logits (to rounding)
    however the prompt is cut and whether rows decode through the hipGraph path or eagerly."""
    m = make(name, "cuda", dtype=torch.bfloat16, seed=9)
    toks = tokens(m, 170 if name == "wide" else 70, 50)
    want = oracle(m).forward(toks)
    whole = replay_alone(m, "cuda", toks, [1000])
    cut = replay_alone(m, "cuda", toks, [7, 1, 2, 1, 1, 16])
    eager = replay_alone(m, "cuda", toks, [30] + [1] * 150, graphs=False)
    for got in (whole, cut, eager):
        check_rounding(got, want)
    check_rounding(cut, whole)


def check_rounding(got, want, rms=2.5e-2, worst=0.12):
    """16-bit activations: the error's root mean square and its maximum over all logits, as
    fractions of the logits' spread."""
    got, want = got.to(ref.F64), want.to(ref.F64)
    scale = max(float(want.std()), 1.0)
    d = got - want
    assert float(d.pow(2).mean().sqrt()) <= rms * scale, f"rms {float(d.pow(2).mean().sqrt()):.3e}"
    assert float(d.abs().max()) <= worst * scale, f"max {float(d.abs().max()):.3e} / {scale:.3f}"


@pytest.mark.gpu
def test_graph_replayed_decode_matches_eager():
    """Decode steps replay a captured hipGraph per batch bucket; several replays, with eager
    prefill steps of other requests between them, give what eager decoding gives."""
    m = make("tiny", "cuda", seed=10)
    a, b = tokens(m, 50, 51), tokens(m, 33, 52)
    wa, wb = oracle(m).forward(a), oracle(m).forward(b)
    rp = TraceReplay(engine(m, "cuda", graphs=True))
    got_a = [rp.step([{"id": "a", "tokens": a[:20], "want": list(range(20))}], [])]
    for i in range(20, 35):                                # graph bucket 1
        got_a.append(rp.step([{"id": "a", "tokens": a[i:i + 1], "want": [0]}], []))
    got_b = [rp.step([{"id": "b", "tokens": b[:10], "want": list(range(10))}], [])]
    for i in range(15):                                    # graph bucket 2, both decoding
        o = rp.step([{"id": "a", "tokens": a[35 + i:36 + i], "want": [0]},
                     {"id": "b", "tokens": b[10 + i:11 + i], "want": [0]}], [])
        got_a.append(o[0:1])
        got_b.append(o[1:2])
    check(torch.cat(got_a, 0), wa)
    check(torch.cat(got_b, 0), wb[:25])
