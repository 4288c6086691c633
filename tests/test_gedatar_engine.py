"""Gedatar through the serving engine (model registry, loader, block manager, state slots,
scheduler, hybrid runner) against the float64 whole-sequence oracle of tests/_ref_gedatar.py.

Every test runs on the CPU (the ops' torch path) and, marked ``gpu``, on the HIP kernels.  The
configurations are small and unlike each other: grouped / multi-query / full-head attention,
chunks smaller than, equal to and unrelated to the cache block size, recurrent heads whose total
size differs from the width, 1 .. 4 conv taps, experts with and without a shared one, top 1 .. 3,
layers without a feed-forward, decay projections of several inner sizes."""
import os

import pytest
import torch

from _ref_gedatar import F64, RefModel

from lumen.models import build_model
from lumen.models.config import ModelConfig, get_config
from lumen.serve.engine import EngineConfig, LLMEngine
from lumen.serve.sequence import SamplingParams
from lumen.serve.trace import TraceReplay

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def _cfg(name, vocab, width, taps, eps, layers):
    return ModelConfig(arch="gedatar", vocab_size=vocab, hidden_size=width, num_hidden_layers=len(layers),
                       rms_norm_eps=eps, canon_taps=taps, intermediate_size=0, num_attention_heads=0,
                       num_key_value_heads=0, max_position_embeddings=1 << 20, eos_token_id=-1,
                       name=name, layer_specs=layers)


def _att(H, G, D, chunk, scale, mlp):
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": scale,
                      "mask": {"size": chunk}}}


def _rec(kind, H, D, mlp):
    return {"type": kind, "mixer": {"heads": H, "dim": D}, "mlp": mlp}


def _moe(E, top, ff, shared):
    m = {"kind": "moe", "router": {"experts": E, "top": top}, "expert": {"ff": ff}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


CONFIGS = {
    "mixed4": lambda: get_config("tiny-gedatar"),
    # multi-query attention with a chunk unrelated to the block size, one recurrent head, top-1
    # routing without a shared expert, a layer without a feed-forward, two taps
    "odd": lambda: _cfg("odd", 97, 64, 2, 3e-6, [
        _rec("general_delta", 1, 64, _moe(3, 1, 40, 0)),
        _att(2, 1, 48, 7, 0.15, {"kind": "dense", "ff": 72}),
        _rec("wkv", 3, 16, None)]),
    # no convolution history at all (one tap), every row its own chunk, all experts chosen
    "edge": lambda: _cfg("edge", 50, 32, 1, 1e-4, [
        _att(2, 2, 16, 1, 0.5, _moe(2, 2, 24, 16)),
        _rec("wkv", 1, 32, {"kind": "dense", "ff": 48}),
        _att(1, 1, 32, 16, 0.2, None)]),
}
RANKS = {"mixed4": 12, "odd": 5, "edge": 16}


def make(name, device, dtype=torch.float32, seed=0):
    from lumen.models.gedatar import GedatarForCausalLM

    cfg = CONFIGS[name]()
    m = GedatarForCausalLM(cfg, dtype=dtype, device=device, decay_rank=RANKS[name])
    m.init_weights(seed=seed)
    return m


def oracle(model):
    return RefModel(model.config, {n: model.tensor(n) for n in model.tensor_names()})


def engine(model, device, blocks=64, bs=16, seqs=4, budget=4096, graphs=True, **kw):
    return LLMEngine(EngineConfig(model=model.config.name, device=device, dtype="fp32" if
                                  model.dtype == torch.float32 else "bf16", num_blocks=blocks,
                                  block_size=bs, max_num_seqs=seqs, max_num_batched_tokens=budget,
                                  max_model_len=blocks * bs, use_graphs=graphs, **kw),
                     model=model, tokenizer=_NoTokenizer())


class _NoTokenizer:
    eos_token_id = None


def tokens(model, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, model.config.vocab_size, (n,), generator=g).tolist()


def check(got, ref, rtol=2e-4):
    got, ref = got.to(F64), ref.to(F64)
    scale = float(ref.std())
    err = float((got - ref).abs().max())
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
    ref = oracle(m).forward(toks)
    check(replay_alone(m, device, toks, [1000]), ref)
    # the model's own forward (fresh state, every row) is the same step function
    check(m(torch.tensor(toks, device=device))[0].cpu(), ref)


@pytest.mark.parametrize("device", DEVICES)
def test_prefill_step_large_enough_for_grouped_experts(device):
    """A 300-row step runs the experts grouped by expert; cut into small steps (and decoding) the
    same tokens run them through the all-experts form.  Both must be the oracle's logits."""
    m = make("mixed4", device, seed=11)
    toks = tokens(m, 300, 12)
    ref = oracle(m).forward(toks)
    check(replay_alone(m, device, toks, [1000]), ref)
    check(replay_alone(m, device, toks, [128, 100, 1]), ref)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_prefill_then_long_decode(device, name):
    """A short prompt, then token by token across several chunk and block borders."""
    m = make(name, device, seed=1)
    toks = tokens(m, 90, 2)
    ref = oracle(m).forward(toks)
    check(replay_alone(m, device, toks, [5] + [1] * 200), ref)
    # from the very first token on, one at a time (the first token is a one-row prefill)
    check(replay_alone(m, device, toks[:40], [1]), ref[:40])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("pieces", [[2], [3, 1, 2, 17, 2, 1, 1, 30], [16], [15, 1, 17]])
def test_portions_of_several_sizes(device, pieces):
    m = make("mixed4", device, seed=2)
    toks = tokens(m, 83, 3)
    check(replay_alone(m, device, toks, pieces, bs=8), oracle(m).forward(toks))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["mixed4", "odd"])
def test_first_tokens(device, name):
    """Sequences shorter than the conv history and the token shift's reach."""
    m = make(name, device, seed=3)
    orc = oracle(m)
    for n in (1, 2, 3):
        toks = tokens(m, n, 10 + n)
        check(replay_alone(m, device, toks, [1000]), orc.forward(toks))
        check(replay_alone(m, device, toks, [1]), orc.forward(toks))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["mixed4", "odd"])
def test_mixed_batches_reuse_blocks_and_slots(device, name):
    """Seven unequal requests through three state slots and a pool of 20 blocks of 8: portions
    of some beside single tokens of others; finished requests hand blocks and slots to new ones.
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
    seen_slots, seen_blocks = [], []
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
        seen_slots += [eng.states.owner.get(rp.live[e["id"]].seq_id) for e in entries
                       if e["id"] in rp.live]
        seen_blocks += [b for t in eng.blocks.tables.values() for b in t]
        o = 0
        for e in entries:
            got[e["id"]].append(out[o:o + len(e["tokens"])])
            o += len(e["tokens"])
    assert len(set(seen_slots) - {None}) <= 3 and eng.states.num_free == 3
    assert eng.blocks.num_free == 20 and len(set(seen_blocks)) <= 20
    for r, toks in reqs.items():
        check(torch.cat(got[r], 0), orc.forward(toks))


@pytest.mark.parametrize("device", DEVICES)
def test_state_slot_and_blocks_reused_after_finish(device):
    """The second request gets the first one's slot and blocks (stale state, stale keys)."""
    m = make("mixed4", device, seed=6)
    orc = oracle(m)
    eng = engine(m, device, blocks=8, bs=16, seqs=1)
    rp = TraceReplay(eng)
    a, b = tokens(m, 100, 30), tokens(m, 60, 31)
    rp.step([{"id": "a", "tokens": a, "want": []}], ["a"])
    got = torch.cat([rp.step([{"id": "b", "tokens": b[:33], "want": list(range(33))}], []),
                     rp.step([{"id": "b", "tokens": b[33:], "want": list(range(27))}], ["b"])], 0)
    check(got, orc.forward(b))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["mixed4", "edge"])
def test_greedy_generation_through_scheduler(device, name):
    """LLMEngine.generate: chunked prefill under a small token budget, more prompts than state
    slots, async scheduling, greedy sampling -- every generated token is the oracle's arg-max
    (up to a tie within the tolerance) given the tokens before it."""
    m = make(name, device, seed=7)
    orc = oracle(m)
    eng = engine(m, device, blocks=48, bs=8, seqs=3, budget=24)
    prompts = [tokens(m, n, 40 + n) for n in (5, 37, 1, 20, 52)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True))
    assert eng.states.num_free == 3 and eng.blocks.num_free == 48
    for p, s in zip(prompts, seqs):
        assert len(s.output_ids) == 10
        ref = orc.forward(p + s.output_ids[:-1])
        for j, tok in enumerate(s.output_ids):
            row = ref[len(p) - 1 + j]
            assert float(row.max() - row[tok]) <= 1e-3 * max(float(row.std()), 1.0)


@pytest.mark.parametrize("device", DEVICES)
def test_preemption_recomputes_state(device):
    """A pool too small for all running sequences: the scheduler preempts and later recomputes a
    sequence from its first token in whatever slot it then gets; outputs stay the oracle's."""
    m = make("odd", device, seed=8)
    orc = oracle(m)
    eng = engine(m, device, blocks=12, bs=4, seqs=3, budget=64, async_scheduling=False)
    prompts = [tokens(m, n, 60 + n) for n in (9, 11, 10)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=14, temperature=0.0, ignore_eos=True))
    assert eng.scheduler.num_preemptions > 0
    for p, s in zip(prompts, seqs):
        ref = orc.forward(p + s.output_ids[:-1])
        for j, tok in enumerate(s.output_ids):
            row = ref[len(p) - 1 + j]
            assert float(row.max() - row[tok]) <= 1e-3 * max(float(row.std()), 1.0)


def test_hybrid_engine_refuses_what_it_cannot_do():
    m = make("edge", "cpu")
    for kw in (dict(enable_prefix_caching=True), dict(num_speculative_tokens=2),
               dict(kv_cache_dtype="fp8")):
        with pytest.raises(ValueError):
            engine(m, "cpu", **kw)


def test_checkpoint_roundtrip_and_strict_names(tmp_path):
    """save -> config.json + model.safetensors under the design's tensor names -> load by
    directory; a missing or an extra tensor is an error."""
    from safetensors.torch import load_file, save_file

    from lumen.models.loading import save_hf_weights

    m = make("odd", "cpu", dtype=torch.bfloat16)
    d = str(tmp_path / "ckpt")
    save_hf_weights(m, d)
    m2 = build_model(d, dtype=torch.bfloat16, device="cpu")
    assert m2.config.arch == "gedatar" and m2.tensor("l0.mix.w1").shape[0] == RANKS["odd"]
    for n in m.tensor_names():
        assert torch.equal(m.tensor(n), m2.tensor(n)), n
    f = os.path.join(d, "model.safetensors")
    sd = load_file(f)
    extra = dict(sd)
    extra["l0.mix.zzz"] = torch.zeros(1)
    save_file(extra, f)
    with pytest.raises(KeyError):
        build_model(d, dtype=torch.bfloat16, device="cpu")
    sd.pop("l1.mix.q")
    save_file(sd, f)
    with pytest.raises(KeyError):
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
def test_bf16_close_to_oracle_and_cut_invariant():
    """bf16 serving: within rounding of the float64 oracle, and the same logits (to rounding)
    however the prompt is cut and whether rows decode through the hipGraph path or eagerly."""
    m = make("mixed4", "cuda", dtype=torch.bfloat16, seed=9)
    toks = tokens(m, 70, 50)
    ref = oracle(m).forward(toks)
    whole = replay_alone(m, "cuda", toks, [1000])
    cut = replay_alone(m, "cuda", toks, [7, 1, 2, 1, 1, 16])
    eager = replay_alone(m, "cuda", toks, [30] + [1] * 50, graphs=False)
    for got in (whole, cut, eager):
        check(got, ref, rtol=6e-2)
    check(cut, whole, rtol=4e-2)
