"""Timisun through the framework (config reader, checkpoint loader, engine, scheduler, paged cache, kernels) against
the plain fp64 definition in timisun_oracle.py. Every scenario runs on the CPU plumbing path in fp32 and, on a GPU
box, through the HIP kernels in fp32 and bf16. Small configurations made here; sizes that differ between layers and
values the obvious choices would make equal or 1 (one head, top 1, window 1, vdim != dim, no shared expert, no
feed-forward, a latent shared with a non-adjacent layer)."""
import json
import os

import numpy as np
import pytest
import torch

import timisun_oracle as oracle
from llmss_amd.engine import LLMEngine, SamplingParams, build_model
from llmss_amd.models.config import ModelConfig
from llmss_amd.models.weights import timisun_state_dict

gpu = pytest.mark.gpu
RUNS = [pytest.param("cpu", "float32", id="cpu-fp32"), pytest.param("cuda", "float32", marks=gpu, id="gpu-fp32"),
        pytest.param("cuda", "bfloat16", marks=gpu, id="gpu-bf16")]


def mixer(heads, dim, vdim, rank, scale, window=None, kv_from=None):
    m = dict(heads=heads, dim=dim, vdim=vdim, kv_rank=rank, scale=scale)
    if window:
        m["mask"] = dict(size=window)
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def moe(experts, top, ff, limit, shared=None):
    d = dict(kind="moe", router=dict(experts=experts, top=top), expert=dict(ff=ff, limit=limit))
    if shared:
        d["shared"] = dict(ff=shared[0], limit=shared[1])
    return d


def layer(m, f=None):
    return dict(type="latent_attention", mixer=m, mlp=f)


CONFIGS = {
    # differing layers; layer 3 reads layer 0's latent (not its neighbour); windows 7 and 20; one layer without ffn
    "mixed": dict(architecture="Timisun", vocab=97, width=40, embedding=dict(scale=3.0), norm=dict(eps=1e-5), layers=[
        layer(mixer(3, 8, 12, 24, 0.35, window=7), moe(6, 2, 24, 2.5, shared=(16, 1.25))),
        layer(mixer(2, 16, 8, 16, 0.25), None),
        layer(mixer(4, 4, 4, 8, 0.5, window=20), moe(3, 3, 8, 1.0)),
        layer(mixer(1, 24, 20, 24, 0.2, window=7, kv_from=0), moe(5, 1, 12, 4.0, shared=(8, 0.5))),
    ]),
    # latent ranks 64 and 128 (in bf16 on a GPU the matrix-core attention kernel runs), windows 33 and 70
    "wide": dict(architecture="Timisun", vocab=83, width=64, embedding=dict(scale=2.0), norm=dict(eps=1e-6), layers=[
        layer(mixer(4, 16, 16, 64, 0.25, window=70), moe(4, 2, 32, 3.0, shared=(32, 2.0))),
        layer(mixer(2, 32, 24, 128, 0.2), None),
        layer(mixer(5, 16, 8, 64, 0.25, window=33, kv_from=0), moe(8, 2, 16, 2.0)),
    ]),
    # one head, top 1, window 1 (a token sees itself only), then a window larger than any test sequence
    "ones": dict(architecture="Timisun", vocab=61, width=24, embedding=dict(scale=1.0), norm=dict(eps=1e-6), layers=[
        layer(mixer(1, 8, 8, 8, 1.0, window=1), moe(2, 1, 8, 1.0)),
        layer(mixer(1, 8, 8, 8, 0.5, window=4096, kv_from=0), moe(2, 2, 8, 1.0, shared=(8, 1.0))),
    ]),
}


class Case:
    def __init__(self, name, tmp, device, dtype, seed=0):
        self.cfg = CONFIGS[name]
        mc = ModelConfig.from_hf_dict(self.cfg)
        self.sd = timisun_state_dict(mc, seed=seed)
        d = tmp / f"{name}-{seed}"
        d.mkdir(exist_ok=True)
        from safetensors.torch import save_file

        sd = dict(self.sd)
        # integer tables stay int32 in a checkpoint; none here. Corrections are stored like everything else.
        save_file({k: v.contiguous() for k, v in sd.items()}, str(d / "model.safetensors"))
        (d / "config.json").write_text(json.dumps(self.cfg))
        self.path, self.device, self.dtype = str(d), device, dtype
        self.model = build_model(self.path, dtype=dtype, device=device)
        self.V = self.cfg["vocab"]
        self._ref = {}

    def engine(self, tokens=512, slots=4, block=16, **kw):
        return LLMEngine(self.model, max_num_seqs=slots, block_size=block, num_blocks=-(-tokens // block),
                         max_model_len=tokens, max_batched_tokens=tokens, use_graphs=kw.pop("use_graphs", False),
                         autotune=False, **kw)

    def ref(self, tokens):
        """Oracle logits [T, V]; in bf16 runs the rows where some router's choice is a close call (the bf16 rounding
        of its input may pick the other expert, which is no fault) are NaN and skipped by close()."""
        key = tuple(tokens)
        if key not in self._ref:
            margins = []
            lg = oracle.forward(self.cfg, self.sd, list(tokens), margins)[0].float()
            if self.dtype != "float32" and margins:
                lg[torch.stack(margins).min(0).values < 0.005] = float("nan")
            self._ref[key] = lg
        return self._ref[key]

    def close(self, got, want, what=""):
        got, want = got.float().cpu(), want.float()
        keep = ~torch.isnan(want).any(-1)
        assert int(keep.sum()) >= 0.5 * len(keep), "too many close calls for a meaningful comparison"
        got, want = got[keep], want[keep]
        d = (got - want) - (got - want).mean(-1, keepdim=True)
        err = d.pow(2).mean(-1).sqrt() / want.std(-1).clamp_min(1e-3)
        tol = 2e-4 if self.dtype == "float32" else 6e-2
        assert float(err.max()) < tol, f"{what}: relative error {float(err.max()):.3g} at row {int(err.argmax())}"


def toks(n, V, seed):
    return np.random.default_rng(seed).integers(0, V, n).tolist()


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("timisun")
    made = {}

    def get(name, device, dtype):
        k = (name, device, dtype)
        if k not in made:
            made[k] = Case(name, tmp, device, dtype)
        return made[k]
    return get


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_every_position(cases, name, device, dtype):
    c = cases(name, device, dtype)
    t = toks(45, c.V, 1)
    eng = c.engine()
    got = eng.replay_step([(0, t, list(range(len(t))))], end=[0])
    c.close(got, c.ref(t), "whole prompt")
    # the first tokens of a sequence on their own: one token, then two
    for n in (1, 2):
        got = eng.replay_step([(n, t[:n], list(range(n)))], end=[n])
        c.close(got, c.ref(t[:n]), f"first {n} token(s)")


@pytest.mark.parametrize("device,dtype", RUNS)
def test_residual_stream_after_every_layer(cases, device, dtype):
    c = cases("mixed", device, dtype)
    t = toks(19, c.V, 2)
    want = oracle.forward(c.cfg, c.sd, t)[1]
    seen = {}
    c.model.tap = lambda i, x: seen.__setitem__(i, x.detach().float().cpu().clone())
    try:
        c.engine().replay_step([(0, t, [len(t) - 1])], end=[0])
    finally:
        c.model.tap = None
    assert sorted(seen) == list(range(len(want)))
    tol = 2e-4 if dtype == "float32" else 5e-2
    for i, w in enumerate(want):
        rel = (seen[i] - w.float()).abs().max() / w.abs().max()
        assert float(rel) < tol, f"layer {i}: {float(rel):.3g}"


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_prefill_against_token_by_token_decoding(cases, name, device, dtype):
    c = cases(name, device, dtype)
    t = toks(40, c.V, 3)
    eng = c.engine()
    rows = [eng.replay_step([(0, [tok], [0])]) for tok in t]  # every token decoded alone, from position 0 on
    eng.replay_step([], end=[0])
    c.close(torch.cat(rows), c.ref(t), "token by token")


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", ["mixed", "wide"])
@pytest.mark.parametrize("cuts", [(2, 2, 2, 3, 5, 16, 17, 2, 1, 1, 9), (15, 1, 16, 1, 17, 6), (33, 2, 21),
                                  (70, 2, 33, 1, 1, 30)])
def test_portions_of_several_sizes(cases, cuts, name, device, dtype):
    c = cases(name, device, dtype)
    t = toks(sum(cuts), c.V, 4)
    eng = c.engine()
    got, at = [], 0
    for n in cuts:
        got.append(eng.replay_step([(7, t[at:at + n], list(range(n)))]))
        at += n
    eng.replay_step([], end=[7])
    c.close(torch.cat(got), c.ref(t), f"portions {cuts}")


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", ["mixed", "wide"])
def test_mixed_batch_of_unequal_requests_equals_each_alone(cases, name, device, dtype):
    c = cases(name, device, dtype)
    seqs = {0: toks(50, c.V, 5), 1: toks(23, c.V, 6), 2: toks(9, c.V, 7), 3: toks(37, c.V, 8)}
    # per step: how many tokens of each request (0 = sits the step out); single tokens ride beside portions
    plan = [{0: 17, 1: 2}, {0: 1, 1: 5, 2: 9}, {0: 1, 1: 16, 3: 30}, {0: 31, 3: 1}, {3: 1, 1: 0}, {3: 5}]
    eng = c.engine(tokens=256)
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    for step in plan:
        entries, end = [], []
        for k, n in step.items():
            if n == 0:
                continue
            entries.append((k, seqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(seqs[k]):
                end.append(k)
        out = eng.replay_step(entries, end)
        r = 0
        for k, tk, _ in entries:
            got[k].append(out[r:r + len(tk)])
            r += len(tk)
    assert at == {k: len(v) for k, v in seqs.items()}
    for k, t in seqs.items():
        c.close(torch.cat(got[k]), c.ref(t), f"request {k} in the mixed batch")


@pytest.mark.parametrize("device,dtype", RUNS)
def test_pages_and_slots_are_used_again(cases, device, dtype):
    c = cases("mixed", device, dtype)
    eng = c.engine(tokens=64, slots=2, block=16)  # 4 pages, 2 sequence slots
    assert eng.sched.num_free_blocks() == 4
    for r in range(6):  # every round takes pages a finished request gave back
        a, b = toks(30 + r, c.V, 10 + r), toks(17, c.V, 20 + r)
        o1 = eng.replay_step([(2 * r, a[:20], [19]), (2 * r + 1, b, [16])], end=[2 * r + 1])
        assert eng.sched.num_free_blocks() == 2
        o2 = eng.replay_step([(2 * r, a[20:], list(range(len(a) - 20)))], end=[2 * r])
        assert eng.sched.num_free_blocks() == 4 and eng.sched.num_running() == 0
        c.close(o1, torch.stack([c.ref(a)[19], c.ref(b)[16]]), f"round {r}, first step")
        c.close(o2, c.ref(a)[20:], f"round {r}, second step")
    with pytest.raises(RuntimeError):  # a third live request has no slot
        eng.replay_step([(100, [1], []), (101, [1], []), (102, [1], [])])
    with pytest.raises(RuntimeError):  # more tokens than the pool has pages for; nothing is taken
        eng.replay_step([(200, [1] * 40, []), (201, [1] * 40, [])])
    assert eng.sched.num_free_blocks() == 4 and eng.sched.num_running() == 0


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", ["mixed", "wide"])
def test_long_decoding_past_every_window(cases, name, device, dtype):
    c = cases(name, device, dtype)
    t = toks(90, c.V, 30)  # every window (7, 20; 33, 70) passes over decoded tokens; pages of 16 are crossed
    eng = c.engine()
    got = [eng.replay_step([(0, t[:5], [4])])]
    got += [eng.replay_step([(0, [tok], [0])]) for tok in t[5:]]
    c.close(torch.cat(got), c.ref(t)[4:], "long decoding")


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_greedy_generation_through_the_engine(cases, name, device, dtype):
    c = cases(name, device, dtype)
    prompts = [toks(11, c.V, 40), toks(3, c.V, 41), toks(26, c.V, 42)]
    eng = LLMEngine(c.model, max_num_seqs=4, block_size=16, num_blocks=32, max_model_len=128, max_batched_tokens=24,
                    prefill_chunk=7, autotune=False)  # its own scheduler cuts the prompts and batches the decodes
    out = eng.generate(prompts, SamplingParams(max_new_tokens=12, is_greedy=True, ignore_eos=True))
    for p, o in zip(prompts, out):
        want = oracle.greedy(c.cfg, c.sd, p, 12)
        if dtype == "float32":
            assert o == want
        else:  # bf16 may flip a near-tie; the tokens before the first difference must then be a true near-tie
            k = next((i for i, (x, y) in enumerate(zip(o, want)) if x != y), None)
            if k is not None:
                lg = oracle.forward(c.cfg, c.sd, p + want[:k])[0][-1]
                assert float(lg[want[k]] - lg[o[k]]) < 0.05 * float(lg.std())


def test_config_reader_rejects_what_the_design_does_not_have():
    bad = json.loads(json.dumps(CONFIGS["ones"]))
    bad["layers"][0]["type"] = "convolution"
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(bad)
    bad = json.loads(json.dumps(CONFIGS["ones"]))
    bad["layers"][1]["mixer"]["kv_from"] = 1  # itself
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(bad)
    bad = json.loads(json.dumps(CONFIGS["ones"]))
    bad["layers"][0]["mlp"]["router"]["top"] = 3  # more than experts
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(bad)


def test_layers_share_one_latent_cache_and_the_pool_counts_owners_only(cases):
    c = cases("mixed", "cpu", "float32")
    kv = c.model.allocate_kv_cache(4, 16)
    assert kv[3][0] is kv[0][0] and kv[1][0] is not kv[0][0]
    assert [k[0].shape[-1] for k in kv] == [24, 16, 8, 24]
    assert c.model.kv_bytes_per_block(16) == 16 * (24 + 16 + 8) * 4


def test_trace_runner_replays_steps_on_the_cpu_path(cases, tmp_path):
    import subprocess
    import sys

    c = cases("ones", "cpu", "float32")
    t = toks(21, c.V, 50)
    steps = [dict(step=0, entries=[dict(id="a", tokens=t[:9], want=[0, 8])], end=[]),
             dict(step=1, entries=[dict(id="b", tokens=t[:2], want=[])], end=[]),
             dict(step=2, entries=[dict(id="a", tokens=t[9:], want=[11]), dict(id="b", tokens=t[2:3], want=[0])],
                  end=["a", "b"])]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", c.path, "--dtype", "float32",
                        "--out", str(tmp_path), "--max-tokens", "64", "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert not os.path.exists(tmp_path / "1.f32")
    g0 = torch.from_numpy(np.fromfile(tmp_path / "0.f32", dtype="<f4").reshape(2, c.V))
    g2 = torch.from_numpy(np.fromfile(tmp_path / "2.f32", dtype="<f4").reshape(2, c.V))
    c.close(g0, c.ref(t)[[0, 8]], "step 0")
    c.close(g2, torch.stack([c.ref(t)[20], c.ref(t[:3])[2]]), "step 2")


def test_registry_facade_runs_the_design(cases):
    """MODEL_REGISTRY["timisun"](config, weights): HF-style calls with a growing paged past."""
    from llmss_amd.models.registry import MODEL_REGISTRY, Weights
    from llmss_amd.utils.checkpoint import weight_files

    c = cases("mixed", "cpu", "float32")
    cfg = ModelConfig.from_pretrained(c.path)
    lm = MODEL_REGISTRY[cfg.model_type](cfg, Weights(weight_files(c.path), "cpu", torch.float32), max_blocks=16)
    t = toks(21, c.V, 60)
    out = lm(torch.tensor([t[:13]]), use_cache=True)
    c.close(out.logits[0], c.ref(t[:13]), "prompt through the facade")
    out2 = lm(torch.tensor([t[13:]]), past_key_values=out.past_key_values, use_cache=True)
    c.close(out2.logits[0], c.ref(t)[13:], "continuation through the facade")
    lm.release(out2.past_key_values)


@gpu
def test_engine_autotunes_the_dense_projections_and_still_decodes_right(cases):
    """With the GEMM autotuner on (the serving default) the plans of the query | latent, output, shared-expert and
    head products are timed per decode bucket; greedy decoding through the captured graphs stays right."""
    c = cases("wide", "cuda", "bfloat16")
    assert c.model.gemm_shapes()
    eng = LLMEngine(c.model, max_num_seqs=2, block_size=16, num_blocks=16, max_model_len=96, max_batched_tokens=64)
    assert eng.tuned and eng.graphs
    p = toks(9, c.V, 70)
    out = eng.generate([p], SamplingParams(max_new_tokens=6, is_greedy=True, ignore_eos=True))[0]
    want = oracle.greedy(c.cfg, c.sd, p, 6)
    k = next((i for i, (x, y) in enumerate(zip(out, want)) if x != y), None)
    if k is not None:
        lg = oracle.forward(c.cfg, c.sd, p + want[:k])[0][-1]
        assert float(lg[want[k]] - lg[out[k]]) < 0.05 * float(lg.std())
