"""The Duparax decoder in the engine against the plain implementation (`plain_duparax`), on the CPU test double
(the engine's logic: batching, cache, state, scheduler) and on the GPU (the kernels, float32 and bfloat16).

Models are tiny and their weights random (`duparax_util.random_weights`); sizes are chosen so that nothing the design
lets differ is equal by accident (dim != vdim on both sides, heads != kv_heads, the two mixers' head counts different,
several blocks, experts of another size than the shared one), with variants where they are equal or 1.
"""

import json

import pytest
import torch

import duparax_util as du
import plain_duparax as plain
from distie_amd import LLM, SamplingParams
from distie_amd.config import ConfigError, config_from_dict, load_model_config
from distie_amd.engine.batch import StepEntry
from distie_amd.engine.model import Model
from torch_ops import TorchOps

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module", params=["cpu", pytest.param("hip", marks=pytest.mark.gpu)])
def ops(request):
    if request.param == "cpu":
        return TorchOps()
    from distie_amd.kernels.hip_ops import HipOps

    return HipOps("cuda:0")


def precisions(ops):
    return ["float32"] if ops.device.type == "cpu" else ["float32", "bfloat16"]


def engine(folder, ops, dtype, **options):
    options.setdefault("block_size", 4 if ops.device.type == "cpu" else 16)
    options.setdefault("num_blocks", 96)
    options.setdefault("max_seqs", 4)
    options.setdefault("use_graphs", False)
    return LLM(folder, dtype=dtype, device=str(ops.device), ops=ops, **options)


def whole(llm, rid, ids):
    out = llm.step([StepEntry(rid, list(ids), list(range(len(ids))))])
    llm.finish(rid)
    return out.float().cpu()


def in_portions(llm, rid, ids, cuts):
    """`ids` in portions of the sizes `cuts`, the rest one token a step; every row's logits."""
    out, at, sizes = [], 0, list(cuts)
    while at < len(ids):
        n = min(sizes.pop(0) if sizes else 1, len(ids) - at)
        out.append(llm.step([StepEntry(rid, list(ids[at:at + n]), list(range(n)))]).float().cpu())
        at += n
    llm.finish(rid)
    return torch.cat(out)


def check(got, want, dtype, what=""):
    """float32: every row within the bound. bfloat16: the norm behind every sub-layer makes a row now and then two or
    three times as sensitive to rounding as the others, so one row in twenty may pass the bound, none 2.5 times it (a
    wrong key, state or expert moves a row by far more)."""
    err = du.logit_error(got, want)
    tol = du.TOL[DTYPES[dtype]]
    worst = f"{what}: error {float(err.max())} at row {int(err.argmax())}"
    if dtype == "float32":
        assert float(err.max()) < tol, worst
    else:
        assert float(err.max()) < 2.5 * tol and int((err > tol).sum()) <= max(1, len(err) // 20), worst


# both kinds of layer and both kinds of feed-forward, nothing equal by accident: keys of 16 and values of 24 on the
# left (a head size of 32 in the kernels), keys of 8 and values of 16 on the right, a temperature step every 5
# positions, four blocks of 16 channels, experts of 24 beside a shared one of 40, a layer without a feed-forward
MIXED = du.make_config([
    du.parallel_layer(heads=4, kv_heads=2, dim=16, vdim=24, coef=0.7, every=5, r_heads=2, r_dim=8, r_vdim=16, tau=4.0, rank=6),
    du.rglru_layer(width=64, blocks=4, conv=4, mlp=du.moe(experts=6, top=2, ff=24, shared=40)),
    du.parallel_layer(heads=6, kv_heads=2, dim=16, vdim=24, coef=0.3, every=7, r_heads=3, r_dim=16, r_vdim=8, tau=9.0,
                      rank=4, mlp=du.moe(experts=5, top=3, ff=16, shared=0)),
    du.rglru_layer(width=48, blocks=3, conv=2, mlp=None),
], vocab=61, width=48, logit_scale=0.4)

# values that the model above makes different made equal, or 1: one head each, dim == vdim == the kernels' head size, no
# temperature, tau 1, one block, a filter of one tap, every expert chosen in one layer and one of them in the
# other, logits not scaled, the recurrent layer in front
PLAIN = du.make_config([
    du.rglru_layer(width=32, blocks=1, conv=1, mlp=du.moe(experts=3, top=3, ff=8, shared=0)),
    du.parallel_layer(heads=1, kv_heads=1, dim=32, vdim=32, every=0, r_heads=1, r_dim=16, r_vdim=16, tau=1.0, rank=1,
                      mlp=du.moe(experts=4, top=1, ff=16, shared=16)),
    du.parallel_layer(heads=2, kv_heads=2, dim=32, vdim=32, coef=1.0, every=1, r_heads=2, r_dim=32, r_vdim=32, tau=2.0,
                      rank=8),
], vocab=40, width=32, logit_scale=None)

# sizes that fit no tile: a width of 40, keys of 20 and values of 12, five heads on one key/value head, blocks of 10
ODD = du.make_config([
    du.parallel_layer(heads=5, kv_heads=1, dim=20, vdim=12, coef=0.5, every=3, r_heads=2, r_dim=12, r_vdim=20, tau=16.0,
                      rank=3, mlp=du.moe(experts=7, top=2, ff=24, shared=8)),
    du.rglru_layer(width=40, blocks=4, conv=3),
], vocab=50, width=40, logit_scale=2.5)

CONFIGS = {"mixed": MIXED, "plain": PLAIN, "odd": ODD}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}
    for name, cfg in CONFIGS.items():
        weights = du.random_weights(cfg, seed=3 + len(made), dtype=torch.bfloat16)
        made[name] = (du.write_model(tmp_path_factory.mktemp(name), cfg, weights), cfg, weights)
    return made


def test_configuration_and_tensors(folders):
    for name, cfg in CONFIGS.items():
        config = config_from_dict(cfg)
        declared = {n: tuple(spec.shape) for n, spec in Model.declare(config.model_spec()).items()}
        assert declared == du.tensor_shapes(cfg)
        # a folder's config.json does not name the decay's rank: the tensors tell it
        read = load_model_config(folders[name][0])
        assert {n: tuple(s.shape) for n, s in Model.declare(read.model_spec()).items()} == du.tensor_shapes(cfg)
    with pytest.raises(ConfigError):
        config_from_dict(du.file_config(MIXED)).model_spec()
    spec = config_from_dict(MIXED).model_spec()
    assert "feed_forward" not in spec.layers[3].parts and spec.head.params["scale"] == 0.4
    for broken in ({**MIXED, "layers": [du.parallel_layer(heads=3, kv_heads=2)]},
                   {**MIXED, "layers": [du.rglru_layer(width=50, blocks=4)]},
                   {**MIXED, "layers": [du.rglru_layer(mlp=du.moe(experts=2, top=3))]},
                   {**MIXED, "layers": [{"type": "other", "mixer": {}, "mlp": None}]},
                   {k: v for k, v in MIXED.items() if k != "norm"}):
        with pytest.raises(ConfigError):
            config_from_dict(broken)


def test_layers_one_by_one(ops, folders):
    """The residual stream behind every layer, through the engine's blocks, against the plain implementation."""
    from distie_amd.parts import ResidualStream, StepContext

    folder, cfg, weights = folders["mixed"]
    ids = du.clear_ids(cfg, weights, 21, seed=1)
    _, after = plain.forward(cfg, weights, ids)
    llm = engine(folder, ops, "float32")
    llm.cache.add("a")
    llm.cache.reserve("a", len(ids))
    tokens, meta, _ = llm.runner.builder.build([StepEntry("a", ids, [0])])
    stream = ResidualStream(llm.model.embed.forward(ops, tokens, meta))
    ctx = StepContext(meta, torch.float32)
    for i, block in enumerate(llm.model.blocks):
        block.forward(ops, stream, ctx, llm.cache.layer(i), True)
        held = stream.hidden.clone()
        delta, post = stream.lanes["pending"]
        ops.add_normed(held, delta, post.weight, post.eps)
        err = (held.double().cpu() - after[i]).abs().max() / after[i].abs().max()
        assert float(err) < 2e-5, f"layer {i}: {float(err)}"


@pytest.mark.parametrize("name", list(CONFIGS))
def test_prompt_decode_and_portions(ops, folders, name):
    """One prompt whole, token by token, and in portions of several sizes down to two tokens: every row's logits
    against the plain implementation, and the same whatever the cut (beyond rounding)."""
    folder, cfg, weights = folders[name]
    ids = du.clear_ids(cfg, weights, 45, seed=11)
    want = du.oracle(cfg, weights, ids)
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype)
        runs = {"whole": whole(llm, "a", ids), "token by token": in_portions(llm, "b", ids, []),
                "portions": in_portions(llm, "c", ids, [2, 7, 3, 2, 13, 5, 2, 4]),
                "a long portion, then tokens": in_portions(llm, "d", ids, [29])}
        for what, got in runs.items():
            check(got, want, dtype, f"{name} {dtype} {what}")
        llm.cache.check()
        assert not llm.cache.live()


def test_unequal_batches_and_reuse(ops, folders):
    """Requests of unequal length side by side, portions beside single tokens, some left out of a step; more requests
    than state slots one after the other, so that pages and slots are used again with what the last owner left."""
    folder, cfg, weights = folders["mixed"]
    prompts = {i: du.clear_ids(cfg, weights, n, seed=20 + i) for i, n in enumerate([31, 6, 19, 2, 40, 1, 23, 12])}
    want = {i: du.oracle(cfg, weights, ids) for i, ids in prompts.items()}
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype, num_blocks=40, max_seqs=3)
        at = {i: 0 for i in prompts}
        got = {i: [] for i in prompts}
        waiting, live, turn = list(prompts), [], 0
        while waiting or live:
            while waiting and len(live) < 3:
                live.append(waiting.pop(0))
            entries = []
            for slot, i in enumerate(live):
                if (turn + slot) % 4 == 3 and len(live) > 1:
                    continue                                  # left out of this step
                left = len(prompts[i]) - at[i]
                n = min(left, [1, 5, 2, 9][(turn + i) % 4])
                entries.append((i, n))
            logits = llm.step([StepEntry(f"r{i}", prompts[i][at[i]:at[i] + n], list(range(n))) for i, n in entries])
            row = 0
            for i, n in entries:
                got[i].append(logits[row:row + n].float().cpu())
                row += n
                at[i] += n
                if at[i] == len(prompts[i]):
                    llm.finish(f"r{i}")
                    live.remove(i)
            llm.cache.check()
            turn += 1
        for i in prompts:
            check(torch.cat(got[i]), want[i], dtype, f"request {i} {dtype}")
        assert not llm.cache.live() and llm.cache.free_pages() == [40] * len(llm.cache.groups)


def planted(cfg, weights, token_a, token_b, strength):
    """Make the key of token `token_a` stand out for queries of token `token_b` in the left mixer of layer 0: a
    direction is added to the key of the normed embedding of a and to the query of that of b, so that their score is
    about `strength` above the others wherever b sees a (before the temperature), and a's value is made large."""
    w = {k: v.clone().float() for k, v in weights.items()}
    m = cfg["layers"][0]["mixer"]["left"]
    D, E, H, G = m["dim"], m["vdim"], m["heads"], m["kv_heads"]
    normed = lambda token: plain.rms_norm(w["embed"][token].double(), w["l0.norm1"].double(), cfg["norm"]["eps"]).float()
    ha, hb = normed(token_a), normed(token_b)
    amount = (strength / float(m["scale"])) ** 0.5
    for g in range(G):
        w["l0.mix.left.k"][g * D:(g + 1) * D] += amount / D ** 0.5 * ha[None, :] / ha.pow(2).sum()
        w["l0.mix.left.v"][g * E:(g + 1) * E] += 3.0 * ha[None, :] / ha.pow(2).sum()
    for h in range(H):
        w["l0.mix.left.q"][h * D:(h + 1) * D] += amount / D ** 0.5 * hb[None, :] / hb.pow(2).sum()
    return {k: v.to(torch.bfloat16) for k, v in w.items()}


FAR = du.make_config([
    du.parallel_layer(heads=2, kv_heads=1, dim=32, vdim=16, scale=0.25, coef=0.5, every=64, r_heads=1, r_dim=16,
                      r_vdim=16, tau=8.0, rank=4, mlp=du.dense(48)),
], vocab=30, width=32)


def test_a_far_key_among_hundreds(ops, tmp_path):
    """Token A's key and value stand out for queries of token B. A lies hundreds of tokens back: the very first token,
    or the last of a page, or the first of the next; B asks for it in a prompt, in a later portion and in decoding.
    A lost or mixed-up page moves the logits there by far more than the tolerance, which the plain implementation
    shows with A taken out."""
    A, B = 7, 11
    weights = planted(FAR, du.random_weights(FAR, seed=9, dtype=torch.float32), A, B, strength=12.0)
    folder = du.write_model(tmp_path / "far", FAR, weights)
    filler = [t for t in du.random_ids(FAR, 900, seed=2) if t not in (A, B)]
    for first in (0, 15, 16, 63, 64):
        ids = filler[:420]
        ids[first] = A
        asks = [first + 1, 200, 255, 256, 300, 383, 384, 385, 419]
        for at in asks:
            ids[at] = B
        want = du.oracle(FAR, weights, ids)
        without = du.oracle(FAR, weights, ids[:first] + [filler[500]] + ids[first + 1:])
        assert float(du.logit_error(without, want)[asks].min()) > 2 * du.TOL[torch.bfloat16]
        for dtype in precisions(ops):
            llm = engine(folder, ops, dtype, block_size=16, num_blocks=30)
            check(whole(llm, "a", ids)[asks], want[asks], dtype, f"prompt, A at {first}, {dtype}")
            got = in_portions(llm, "b", ids, [first + 1, 2, 197 - first, 56, 2, 120])
            check(got[asks], want[asks], dtype, f"portions, then decoding, A at {first}, {dtype}")


def test_temperature_steps(ops, folders):
    """The query temperature changes at every multiple of `every`: the tokens around those places, in a prompt, at
    the start of a portion and decoded alone. Other steps show in the plain implementation at most places."""
    folder, cfg, weights = folders["plain"]             # its last layer steps at every position, with coef 1
    ids = du.clear_ids(cfg, weights, 40, seed=3)
    want = du.oracle(cfg, weights, ids)
    shifted = json.loads(json.dumps(cfg))
    shifted["layers"][2]["mixer"]["left"]["q_temp"]["every"] = 2
    assert float(du.logit_error(du.oracle(shifted, weights, ids), want)[1:].median()) > 10 * du.TOL[torch.float32]
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype)
        check(in_portions(llm, "a", ids, [1, 1, 2, 3, 4, 9, 10]), want, dtype, f"every position {dtype}")


def test_far_state_reaches_the_present(ops, tmp_path):
    """Slow decays in both kinds of state: what the first token wrote still shows hundreds of tokens later, through a
    prompt in one piece, in portions and in decoding (the states are carried, not recomputed). Shown by the plain
    implementation on the same tokens with another first token."""
    for kind in ("gated", "recurrent"):
        if kind == "gated":
            cfg = du.make_config([du.parallel_layer(heads=1, kv_heads=1, dim=16, vdim=16, every=0, r_heads=2, r_dim=16,
                                                    r_vdim=16, tau=64.0, rank=4, mlp=None)], vocab=30, width=32)
        else:
            cfg = du.make_config([du.rglru_layer(width=32, blocks=2, conv=3, mlp=None)], vocab=30, width=32)
        weights = du.random_weights(cfg, seed=4, dtype=torch.float32)
        if kind == "gated":
            weights["l0.mix.right.a2.b"] += 4.0                  # decays close to one
            weights["l0.mix.left.o"] *= 0.05                     # the attention beside it must not drown the state
        else:
            weights["l0.mix.lam"] -= 7.0
        weights = {k: v.to(torch.bfloat16) for k, v in weights.items()}
        ids = du.clear_ids(cfg, weights, 6, seed=8) + du.random_ids(cfg, 254, seed=8)     # no close call at the start
        want = du.oracle(cfg, weights, ids)
        other = du.oracle(cfg, weights, [(ids[0] + 1) % 30] + ids[1:])
        assert float(du.logit_error(other[-5:], want[-5:]).min()) > 10 * du.TOL[torch.float32], kind
        folder = du.write_model(tmp_path / kind, cfg, weights)
        for dtype in precisions(ops):
            llm = engine(folder, ops, dtype)
            check(whole(llm, "a", ids)[-40:], want[-40:], dtype, f"{kind} whole {dtype}")
            check(in_portions(llm, "b", ids, [64, 2, 100, 61])[-40:], want[-40:], dtype, f"{kind} portions {dtype}")


def test_greedy_generation_through_the_scheduler(ops, folders):
    """`LLM.generate`: continuous batching with a token budget that cuts the prompts, more requests than seats, and
    (on the GPU) captured decode steps. Every token is the plain implementation's greedy pick given what came before,
    or a near tie. bfloat16 on a model whose routing does not hang on a close call (every expert chosen)."""
    for name, dtypes in (("mixed", ["float32"]), ("plain", precisions(ops))):
        folder, cfg, weights = folders[name]
        if name == "plain":
            cfg = json.loads(json.dumps(cfg))
            cfg["layers"] = [cfg["layers"][0], cfg["layers"][2]]
            weights = {("l1." + n[3:] if n.startswith("l2.") else n): t for n, t in weights.items() if not n.startswith("l1.")}
            folder = du.write_model(folder / "dense", cfg, weights)
        prompts = [du.random_ids(cfg, n, seed=40 + n) for n in (23, 5, 14, 9, 2)]
        for dtype in dtypes:
            llm = engine(folder, ops, dtype, num_blocks=64, max_seqs=3, token_budget=16,
                         use_graphs=ops.device.type != "cpu")
            outs = llm.generate(prompts, SamplingParams(max_new_tokens=12))
            slack = 1e-3 if dtype == "float32" else 0.35
            for prompt, out in zip(prompts, outs):
                assert len(out.token_ids) == 12
                ids = list(prompt)
                for token in out.token_ids:
                    logits = du.oracle(cfg, weights, ids)[-1]
                    assert float(logits[token]) >= float(logits.max()) - slack * float(logits.abs().max()), (dtype, out.token_ids)
                    ids.append(token)
            assert not llm.cache.live()
            llm.close()


def test_random_model_folder_reads_back(tmp_path):
    """`random-model` of the command line writes a folder that the loader takes, tensor for tensor as the design
    names them."""
    from distie_amd import cli
    from distie_amd.weights.safetensors_io import SafetensorsFile

    (tmp_path / "config.json").write_text(json.dumps(PLAIN))
    assert cli.main(["random-model", "--config-json", str(tmp_path / "config.json"), "--out", str(tmp_path / "m"),
                     "--seed", "3", "--dtype", "bf16", "--std", "0.1"]) == 0
    stored = SafetensorsFile(tmp_path / "m" / "model.safetensors")
    assert {name: tuple(entry[1]) for name, entry in stored.index.items()} == du.tensor_shapes(PLAIN)
    stored.close()
    llm = engine(tmp_path / "m", TorchOps(), "float32")
    assert llm.step([StepEntry("a", [1, 2, 3], [2])]).shape == (1, PLAIN["vocab"])


@pytest.mark.gpu
def test_trace_runner_and_command_line(folders, tmp_path):
    """The trace runner as a program (its own process, steps on standard input, four requests live, pages and
    slots used again) and `generate` of the command line, on a Duparax model, against the plain implementation."""
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parents[1]
    folder, cfg, weights = folders["mixed"]
    lengths = {"p": 70, "q": 33, "r": 64, "s": 5, "t": 50, "u": 21}
    reqs = {r: du.clear_ids(cfg, weights, n, 60 + n) for r, n in lengths.items()}
    want = {r: du.oracle(cfg, weights, ids) for r, ids in reqs.items()}
    max_tokens = sum(-(-n // 64) * 64 for n in sorted(lengths.values())[-4:])
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / dtype
        proc = subprocess.Popen([sys.executable, str(root / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype,
                                 "--out", str(out), "--max-tokens", str(max_tokens)],
                                stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
        got, at = {r: [] for r in reqs}, {r: 0 for r in reqs}
        waiting, live, step = list(reqs), [], 0
        while waiting or live:
            while waiting and len(live) < 4:
                live.append(waiting.pop(0))
            entries, end = [], []
            for k, r in enumerate(live):
                left = len(reqs[r]) - at[r]
                n = min(left, 1 if left <= 8 else [13, 2, 30, 7][(step + k) % 4])
                entries.append({"id": r, "tokens": reqs[r][at[r]:at[r] + n], "want": list(range(n))})
                at[r] += n
                if at[r] == len(reqs[r]):
                    end.append(r)
            proc.stdin.write(json.dumps({"step": step, "entries": entries, "end": end}) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {step}"
            rows = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, cfg["vocab"]).copy())
            row = 0
            for e in entries:
                got[e["id"]].append(rows[row:row + len(e["tokens"])])
                row += len(e["tokens"])
            live = [r for r in live if r not in end]
            step += 1
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
        for r in reqs:
            check(torch.cat(got[r]), want[r], dtype, f"request {r} {dtype}")
    prompts = [reqs["s"], reqs["q"][:9]]
    (tmp_path / "prompts.json").write_text(json.dumps(prompts))
    done = subprocess.run([sys.executable, "-m", "distie_amd.cli", "generate", "--model", str(folder), "--dtype", "fp32",
                           "--prompts", str(tmp_path / "prompts.json"), "--max-new-tokens", "6", "--num-blocks", "32",
                           "--out", str(tmp_path / "report.json")], cwd=str(root), capture_output=True, text=True, timeout=110)
    assert done.returncode == 0, done.stderr
    for prompt, record in zip(prompts, json.loads((tmp_path / "report.json").read_text())):
        ids = list(prompt)
        for token in record["token_ids"]:
            logits = du.oracle(cfg, weights, ids)[-1]
            assert float(logits[token]) >= float(logits.max()) - 1e-3 * float(logits.abs().max())
            ids.append(token)


def test_preemption_starts_the_state_over(ops, folders):
    """So few pages that running requests are preempted and recomputed: their convolution inputs and both kinds of
    state start from zero again, and every token still is the plain implementation's pick."""
    folder, cfg, weights = folders["mixed"]
    prompts = [du.random_ids(cfg, n, seed=70 + n) for n in (20, 26, 17)]
    block = 4 if ops.device.type == "cpu" else 16
    new = 24 if block == 4 else 40
    # as many pages as the longest request may hold by itself: three of them do not fit side by side
    llm = engine(folder, ops, "float32", block_size=block, num_blocks=-(-(26 + new) // block) + 1, max_seqs=3, token_budget=32)
    outs = llm.generate(prompts, SamplingParams(max_new_tokens=new))
    assert sum(o.preemptions for o in outs) > 0, "the pool was not small enough to preempt anybody"
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for token in out.token_ids:
            logits = du.oracle(cfg, weights, ids)[-1]
            assert float(logits[token]) >= float(logits.max()) - 1e-3 * float(logits.abs().max())
            ids.append(token)
    llm.cache.check()
    assert not llm.cache.live()
