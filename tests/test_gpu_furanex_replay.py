"""Furanex in the engine against the plain model under every way of cutting the same requests:
whole, last tokens one by one (through graphs and without), portions of changing size down to two
tokens, mixed with other requests on so few pages and slots that they are used again; float32 and
bfloat16; small configurations that differ in every size and option (stream counts, layer orders,
head and latent sizes, rotated channels, stretches, experts a token, shared experts or none); and
greedy generation through the engine's own entry point and scheduler."""
import numpy as np
import pytest
import torch

import trace_tools
from furanex_helpers import (FUR, make_weights, plain_logits, plain_logits_bf16, plain_logits_f32, random_tokens, sharpened)
from helpers import TOL_F32, bf16_tolerance, rel_err, write_model_dir

pytestmark = pytest.mark.gpu

NAMES = ["A", "B", "C", "D", "E"]
LENGTHS = {"A": [70, 5, 45, 21, 33, 2], "B": [88, 40, 66, 3, 58], "C": [150, 17, 230, 49], "D": [50, 36, 77, 1],
           "E": [40, 3, 65, 129]}
PAGE = {"A": 16, "B": 8, "C": 16, "D": 16, "E": 8}
GAINS = {"sharp": 12.0, "mild": 1.0}
# q and k are unit vectors, so a score is at most scale x dim: the heads of 64 and 128 channels of C get a smaller factor
# (their largest score is then 26 instead of 77, beyond which bfloat16 rounding of the cached keys alone moves the logits
# by a tenth)
SHARP_OF = {"C": 4.0}


def judge(errors, tol, dtype, what):
    """Every row within the tolerance: the experts of a token are named by a table, so no choice can fall the
    other way, and nothing is set aside."""
    worst = max(errors) if errors else 0.0
    print(f"{what} [{dtype}]: {len(errors)} rows, worst relative error {worst:.3e} (allowed {tol:.3e})")
    assert worst <= tol, f"{what}: relative error {worst:.3e} exceeds {tol:.1e}"


class Case:
    def __init__(self, name, tmp, kind):
        self.name, self.kind, self.page = name, kind, PAGE[name]
        self.cfg = sharpened(FUR[name], SHARP_OF.get(name, GAINS[kind]) if kind == "sharp" else GAINS[kind])
        self.weights = make_weights(self.cfg, seed=sum(map(ord, name)) + 1, key_gain=2.0 if kind == "sharp" else 1.0)
        self.dir = write_model_dir(str(tmp / f"fur{name}_{kind}"), self.cfg, self.weights)
        self.reqs = {f"r{i}": random_tokens(self.cfg, n, seed=100 + i) for i, n in enumerate(LENGTHS[name])}
        self.want = {rid: plain_logits(self.cfg, self.weights, toks) for rid, toks in self.reqs.items()}
        emulated = {rid: plain_logits_bf16(self.cfg, self.weights, toks) for rid, toks in self.reqs.items()}
        self.bf16_error = max(rel_err(emulated[rid][p], self.want[rid][p])
                              for rid, toks in self.reqs.items() for p in range(len(toks)))
        single = {rid: plain_logits_f32(self.cfg, self.weights, toks) for rid, toks in self.reqs.items()}
        self.f32_error = max(rel_err(single[rid][p], self.want[rid][p])
                             for rid, toks in self.reqs.items() for p in range(len(toks)))

    def tol(self, dtype):
        # float32: the usual bound, or eight times what 32-bit arithmetic alone does to the plain model
        return max(TOL_F32, 8 * self.f32_error) if dtype == "float32" else bf16_tolerance(self.bf16_error)

    def check(self, got, dtype, what):
        judge([rel_err(row, self.want[rid][pos]) for (rid, pos), row in got.items()], self.tol(dtype), dtype, what)
        return sum(len(t) for t in self.reqs.values())


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("furanex")
    return {(name, kind): Case(name, tmp, kind) for name in NAMES for kind in GAINS}


def runner_for(case, dtype, steps, page_size=None, use_graph=True, **kw):
    from minivllm_amd.engine.trace import TraceRunner
    return TraceRunner(case.dir, dtype, trace_tools.max_live_tokens(steps), page_size=page_size or case.page,
                       use_graph=use_graph, **kw)


def both(cases, name):
    return [cases[(name, kind)] for kind in GAINS]


def prompt_lens_of(case):
    return {rid: max(2, len(t) - 12) if len(t) > 3 else len(t) for rid, t in case.reqs.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_whole(cases, name, dtype):
    for case in both(cases, name):
        steps = trace_tools.whole(case.reqs)
        got = trace_tools.collect(steps, runner_for(case, dtype, steps).run_step)
        assert len(got) == case.check(got, dtype, f"{name} {case.kind} whole")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("use_graph", [True, False])
def test_tail_decode(cases, name, dtype, use_graph):
    """The last 40 tokens one by one, from the cache that the prompt left: the values blended with the first
    layer's are those of the step's own token."""
    case = cases[(name, "sharp")]
    steps = trace_tools.tail_decode(case.reqs, tail=40)
    got = trace_tools.collect(steps, runner_for(case, dtype, steps, use_graph=use_graph).run_step)
    case.check(got, dtype, f"{name} last 40 one by one (graph={use_graph})")
    assert all((rid, len(toks) - 1) in got for rid, toks in case.reqs.items())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("page_size", ["own", 4])
def test_portions(cases, name, dtype, page_size):
    """Portions of 7, 5, 3, 2, 11, 2, 17, 2, 4 tokens, across pages."""
    case = cases[(name, "sharp")]
    steps = trace_tools.portions(case.reqs)
    ps = case.page if page_size == "own" else page_size
    got = trace_tools.collect(steps, runner_for(case, dtype, steps, page_size=ps).run_step)
    assert len(got) == case.check(got, dtype, f"{name} portions (page {ps})")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_mixed(cases, name, dtype):
    """Up to three live requests on three slots and pages for exactly the live tokens: pages change hands, and a row's
    experts follow its own token id whatever stands beside it in the step."""
    for case in both(cases, name):
        for seed in (0, 1):
            steps = trace_tools.mixed(case.reqs, prompt_lens_of(case), max_live=3, seed=seed)
            runner = runner_for(case, dtype, steps, max_live=3)
            got = trace_tools.collect(steps, runner.run_step)
            assert len(got) == case.check(got, dtype, f"{name} {case.kind} mixed seed {seed}")
            runner.manager.check_invariants()
            assert not runner.manager.seqs and runner.manager.slots.num_free == 3
            for pool in runner.manager.pools:
                assert pool.num_free == pool.num_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_steps_with_prompt_portions_from_graphs(cases, name, dtype):
    """Every entry wants its last row only, as generation does: such steps are replayed from graphs per size class,
    padded with inert rows (whose token ids still name experts) and sequences."""
    case = cases[(name, "sharp")]
    cuttings = {"portions": trace_tools.portions(case.reqs),
                "mixed": trace_tools.mixed(case.reqs, prompt_lens_of(case), max_live=4, seed=4)}
    for what, steps in cuttings.items():
        steps = trace_tools.only_last_rows(steps)
        runner = runner_for(case, dtype, steps)
        got = trace_tools.collect(steps, runner.run_step)
        case.check(got, dtype, f"{name} {what} from graphs")
        assert len(got) == sum(len(st["entries"]) for st in steps)
        assert runner.executor.model.graph_safe and list(runner.executor._mixed_graphs)
        eager = trace_tools.collect(steps, runner_for(case, dtype, steps, use_graph=False).run_step)
        judge([rel_err(got[k], eager[k]) for k in got], 1e-6 if dtype == "float32" else 2e-2, dtype, "graphs against eager steps")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C", "D"])
def test_mixed_with_poisoned_pages(cases, name, dtype):
    """Pages are filled with NaN when they change hands: a kernel that reads a slot nobody has written since puts NaN
    into the logits."""
    case = cases[(name, "sharp")]
    steps = trace_tools.mixed(case.reqs, prompt_lens_of(case), max_live=4, seed=2)
    runner = runner_for(case, dtype, steps, poison_pages=True)
    got = trace_tools.collect(steps, runner.run_step)
    assert len(got) == case.check(got, dtype, f"{name} mixed on poisoned pages")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens_and_short_requests(cases, name, dtype):
    case = cases[(name, "sharp")]
    reqs = {"one": case.reqs["r0"][:1], "two": case.reqs["r0"][:2], "three": case.reqs["r1"][:3]}
    steps = trace_tools.whole(reqs) + [dict(st, step=st["step"] + 3) for st in trace_tools.tail_decode(
        {"again": case.reqs["r0"][:6]}, tail=5)]
    got = trace_tools.collect(steps, runner_for(case, dtype, steps).run_step)
    assert len(got) == 1 + 2 + 3 + 6
    judge([rel_err(row, case.want["r1" if rid == "three" else "r0"][pos]) for (rid, pos), row in got.items()], case.tol(dtype),
          dtype, "first tokens")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C", "E"])
def test_long_decoding(cases, name, dtype):
    """Four tokens of prompt, then 250 tokens one by one."""
    case = cases[(name, "mild")]
    toks = random_tokens(case.cfg, 254, seed=9)
    want = plain_logits(case.cfg, case.weights, toks)
    steps = trace_tools.tail_decode({"long": toks}, tail=250)
    got = trace_tools.collect(steps, runner_for(case, dtype, steps).run_step)
    tol = TOL_F32 if dtype == "float32" else bf16_tolerance(
        max(rel_err(a, b) for a, b in zip(plain_logits_bf16(case.cfg, case.weights, toks), want)))
    assert len(got) == 251
    judge([rel_err(row, want[pos]) for (_, pos), row in got.items()], tol, dtype, f"{name} long decoding")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation(cases, name, dtype):
    """Through LLM.generate: the scheduler cuts prompts into portions of at most 24 tokens, batches them with decoding
    requests, runs decode steps in rows from graphs, and preempts when pages run out."""
    from minivllm_amd import LLM, SamplingParams
    case = cases[(name, "mild")]
    llm = LLM(model=case.dir, dtype=dtype, kv_cache_block_size=case.page, kv_cache_num_blocks=40, max_model_len=320,
              max_num_batched_tokens=48, max_num_batched_seqs=4, prefill_chunk=24)
    prompts = [random_tokens(case.cfg, n, seed=n) for n in (5, 61, 33, 1, 90, 18)]
    sp = SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True)
    outs = llm.generate(prompts, sp, use_tqdm=False)
    assert [o.prompt_token_ids for o in outs] == prompts and all(len(o.token_ids) == 40 for o in outs)
    clear = near = 0
    for out in outs:
        seq = list(out.prompt_token_ids) + list(out.token_ids)
        logits = plain_logits(case.cfg, case.weights, seq)
        tol = TOL_F32 if dtype == "float32" else bf16_tolerance(
            max(rel_err(a, b) for a, b in zip(plain_logits_bf16(case.cfg, case.weights, seq), logits)))
        for t, tok in enumerate(out.token_ids):
            row = logits[len(out.prompt_token_ids) + t - 1]
            slack = 2 * tol * float(np.abs(row).max())
            assert row[tok] >= row.max() - slack, f"token {t}: {tok} scores {row[tok]}, the best {row.max()}"
            if row.max() - np.partition(row, -2)[-2] > slack:
                assert tok == int(row.argmax())
                clear += 1
            else:
                near += 1
    print(f"greedy {name} [{dtype}]: {clear} tokens decided by a clear margin, {near} near ties")
    assert clear > near if dtype == "float32" else True
    llm.manager.check_invariants()


def test_command_lines(cases, tmp_path):
    """``run.py --random-model furanex-tiny`` prints completions, and ``bin/trace_run`` as a program, fed a trace on its
    standard input, writes the logits the plain model gives (four state slots by default)."""
    import ast
    import json
    import os
    import re
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "run.py"), "--random-model", "furanex-tiny", "--seed", "3",
                           "--prompt-ids", "5,17,3", "--prompt-ids", "200", "--max-tokens", "5", "--temperature", "0",
                           "--ignore-eos", "--max-model-len", "64", "--kv-cache-num-blocks", "16",
                           "--max-num-batched-tokens", "64", "--max-num-batched-seqs", "4"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    completions = re.findall(r"Completion:\s*(\[.*?\])", proc.stdout, re.S)
    assert len(completions) == 2 and all(len(ast.literal_eval(c)) == 5 for c in completions)

    case = cases[("D", "mild")]
    steps = trace_tools.mixed(case.reqs, prompt_lens_of(case), max_live=4, seed=7)
    out = tmp_path / "logits"
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", case.dir, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", str(trace_tools.max_live_tokens(steps))],
                          input="".join(json.dumps(st) + "\n" for st in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done ")] == [f"done {st['step']}" for st in steps]
    got = trace_tools.collect(steps, lambda st: (np.fromfile(out / f"{st['step']}.f32", dtype="<f4").reshape(
        -1, case.cfg["vocab"]) if any(e["want"] for e in st["entries"]) else None))
    case.check(got, "float32", "D mixed through bin/trace_run")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_request_past_a_thousand_tokens(cases, dtype):
    """1,100 tokens through sizes that resemble a real model's heads: whole, and the last 40 tokens one by one behind a
    prompt fed in two portions; positions far beyond the length the stretched frequencies were made for."""
    case = cases[("C", "mild")]
    toks = random_tokens(case.cfg, 1100, seed=77)
    want = plain_logits(case.cfg, case.weights, toks)
    rows = [0, 1, 47, 48, 511, 512, 1023, 1024, 1059, 1060, 1099]
    tol = TOL_F32 if dtype == "float32" else bf16_tolerance(
        max(rel_err(plain_logits_bf16(case.cfg, case.weights, toks)[p], want[p]) for p in rows))
    steps = [{"step": 0, "entries": [{"id": "w", "tokens": toks, "want": rows}], "end": ["w"]},
             {"step": 1, "entries": [{"id": "d", "tokens": toks[:1000], "want": [999]}], "end": []},
             {"step": 2, "entries": [{"id": "d", "tokens": toks[1000:1060], "want": [59]}], "end": []}]
    steps += [{"step": 3 + i, "entries": [{"id": "d", "tokens": [toks[1060 + i]], "want": [0]}],
               "end": ["d"] if i == 39 else []} for i in range(40)]
    got = trace_tools.collect(steps, runner_for(case, dtype, steps).run_step)
    assert len(got) == len(rows) + 2 + 40
    judge([rel_err(row, want[pos]) for (_, pos), row in got.items()], tol, dtype, "1,100 tokens")


@pytest.mark.parametrize("seed, fast_sizes", [(21, False), (22, False), (23, True), (24, True), (25, False)])
def test_configurations_drawn_at_random(tmp_path, seed, fast_sizes):
    """Sizes nobody chose: every size and option drawn at random, five requests (one of them past 1,024 tokens) mixed on
    four slots in portions of up to 130 tokens, float32 and bfloat16."""
    from furanex_helpers import random_config
    from minivllm_amd.engine.trace import TraceRunner
    rng = np.random.default_rng(seed)
    cfg = random_config(rng, fast_sizes=fast_sizes)
    weights = make_weights(cfg, seed=seed)
    model = write_model_dir(str(tmp_path / "m"), cfg, weights)
    lens = [int(x) for x in rng.integers(1, 200, size=4)] + [1100]
    reqs = {f"r{i}": random_tokens(cfg, n, seed=i) for i, n in enumerate(lens)}
    want = {rid: plain_logits(cfg, weights, toks) for rid, toks in reqs.items()}
    sample = [(rid, p) for rid, toks in reqs.items() for p in range(0, len(toks), 7)]
    single = {rid: plain_logits_f32(cfg, weights, toks) for rid, toks in reqs.items()}
    f32_error = max(rel_err(single[rid][p], want[rid][p]) for rid, toks in reqs.items() for p in range(len(toks)))
    steps = trace_tools.mixed(reqs, {rid: max(2, len(t) - 12) if len(t) > 3 else len(t) for rid, t in reqs.items()}, max_live=4,
                              seed=seed, max_portion=130)
    for dtype in ["float32", "bfloat16"]:
        got = trace_tools.collect(steps, TraceRunner(model, dtype, trace_tools.max_live_tokens(steps), page_size=16,
                                                     max_live=4).run_step)
        assert len(got) == sum(lens)
        if dtype == "float32":
            tol = max(TOL_F32, 8 * f32_error)
        else:
            tol = bf16_tolerance(max(rel_err(plain_logits_bf16(cfg, weights, reqs[rid])[p], want[rid][p]) for rid, p in sample))
        judge([rel_err(row, want[rid][pos]) for (rid, pos), row in got.items()], tol, dtype, f"random configuration {seed}")


@pytest.mark.parametrize("name", ["A", "B"])
def test_sizes_left_out_of_the_configuration(cases, tmp_path, name):
    """A folder whose config.json leaves out everything the stored tensors' shapes state serves like the full one."""
    import copy
    case = cases[(name, "mild")]
    raw = copy.deepcopy(case.cfg)
    for key in ("vocab", "width", "streams"):
        raw.pop(key, None)
    for layer in raw["layers"]:
        for key in ("heads", "kv_heads", "vdim", "q_rank", "kv_rank", "rot_dim"):
            layer["mixer"].pop(key, None)
        if layer["type"] == "latent_attention":
            layer["mixer"].pop("dim")
        if layer.get("mlp"):
            layer["mlp"] = {"kind": "moe"}
    thin = type("Thin", (), {"dir": write_model_dir(str(tmp_path / "thin"), raw, case.weights), "page": case.page})()
    steps = trace_tools.portions(case.reqs)
    got = trace_tools.collect(steps, runner_for(thin, "float32", steps).run_step)
    assert len(got) == case.check(got, "float32", f"{name} with sizes left out")
