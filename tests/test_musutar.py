"""The Musutar decoder in the engine against the plain implementation (`plain_musutar`), on the CPU test double
(the engine's logic: batching, cache, state, scheduler) and on the GPU (the kernels, float32 and bfloat16).

Models are tiny and their weights random (`musutar_util.random_weights`); sizes are chosen so that nothing the
design lets differ is equal by accident (dim != vdim, rotated dims < dim, heads != kv_heads, streams 1/2/3, taps of
the two convolutions different), with variants where they are equal or 1.
"""

import torch
import pytest

import musutar_util as mu
import plain_musutar as plain
from distie_amd import LLM, SamplingParams
from distie_amd.config import ConfigError, config_from_dict
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
    err = mu.logit_error(got, want)
    assert float(err.max()) < mu.TOL[DTYPES[dtype]], f"{what}: error {float(err.max())} at row {int(err.argmax())}"


# the design's mixers side by side, nothing equal by accident: keys of 16 and values of 24 (a head size of 32 in the
# kernels), 8 of 16 dimensions rotated with scaled frequencies, a window of 12 that two later layers borrow with
# windows of their own, a layer without a feed-forward, a state mixer with keys of 8 and values of 16
MIXED = mu.make_config([
    mu.attention_layer(heads=4, kv_heads=2, dim=16, vdim=24, conv=4, window=12, rot_dims=8),
    mu.lightning_layer(heads=2, dim=8, vdim=16, decay=(0.7, 0.97)),
    mu.attention_layer(heads=4, kv_heads=2, dim=16, vdim=24, conv=4, window=9, rot_dims=8, kv_from=0, ff=0),
    mu.attention_layer(heads=6, kv_heads=2, dim=16, vdim=24, conv=2, window=17, rot_dims=8, kv_from=0, ff=40),
    mu.lightning_layer(heads=3, dim=16, vdim=8, decay=(0.5, 0.9, 0.999), ff=56),
], vocab=61, width=48, streams=2, taps=3)

# values that the model above makes different made equal, or 1: one stream, one kv head for every head, dim == vdim
# == rotated dims, no scaling, filters of one tap, no window, a state mixer in front
PLAIN = mu.make_config([
    mu.lightning_layer(heads=1, dim=16, vdim=16, decay=(0.9,), ff=0),
    mu.attention_layer(heads=2, kv_heads=2, dim=32, vdim=32, conv=1, window=None, rot_dims=32, scaling=False, scale=0.2),
    mu.attention_layer(heads=2, kv_heads=2, dim=32, vdim=32, conv=1, window=5, rot_dims=32, scaling=False, kv_from=1),
], vocab=40, width=32, streams=1, taps=1)

# three streams, no convolutions at all, no rotation, wide heads
BARE = mu.make_config([
    mu.attention_layer(heads=2, kv_heads=1, dim=40, vdim=64, conv=0, window=7, rot_dims=0, scale=0.15, ff=64),
    mu.lightning_layer(heads=2, dim=24, vdim=24, decay=(0.8, 0.95), ff=64),
], vocab=50, width=64, streams=3, taps=0)

CONFIGS = {"mixed": MIXED, "plain": PLAIN, "bare": BARE}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}
    for name, cfg in CONFIGS.items():
        weights = mu.random_weights(cfg, seed=3 + len(made), dtype=torch.bfloat16)
        made[name] = (mu.write_model(tmp_path_factory.mktemp(name), cfg, weights), cfg, weights)
    return made


def test_configuration_and_tensors():
    for cfg in CONFIGS.values():
        config = config_from_dict(cfg)
        declared = {name: tuple(spec.shape) for name, spec in Model.declare(config.model_spec()).items()}
        assert declared == mu.tensor_shapes(cfg)
    spec = config_from_dict(MIXED).model_spec()
    assert spec.layers[0].parts["mixer"].params["keep"] == 17       # the widest window among lender and borrowers
    assert "feed_forward" not in spec.layers[2].parts
    for broken in ({**MIXED, "layers": [mu.attention_layer(kv_from=0)]},
                   {**MIXED, "layers": [mu.lightning_layer(decay=(0.5,))]},
                   {**MIXED, "layers": [{"type": "other", "mixer": {"heads": 1, "dim": 2, "vdim": 2}, "mlp": None}]},
                   {k: v for k, v in MIXED.items() if k != "norm"}):
        with pytest.raises(ConfigError):
            config_from_dict(broken)


@pytest.mark.parametrize("name", list(CONFIGS))
def test_prompt_decode_and_portions(ops, folders, name):
    """One prompt whole, token by token, and in portions of several sizes down to two tokens: every row's logits
    against the plain implementation, and the same whatever the cut (beyond rounding)."""
    folder, cfg, weights = folders[name]
    ids = mu.random_ids(cfg, 45, seed=11)
    want = mu.oracle(cfg, weights, ids)
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
    prompts = {i: mu.random_ids(cfg, n, seed=20 + i) for i, n in enumerate([31, 6, 19, 2, 40, 1, 23, 12])}
    want = {i: mu.oracle(cfg, weights, ids) for i, ids in prompts.items()}
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


def test_long_decoding_past_every_window(ops, folders):
    """A short prompt and then many single tokens: every window passes over decoded tokens, pages of the windowed
    group are given back on the way, the decayed state carries on."""
    folder, cfg, weights = folders["mixed"]
    ids = mu.random_ids(cfg, 70, seed=5)
    want = mu.oracle(cfg, weights, ids)
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype, num_blocks=16)
        got = in_portions(llm, "a", ids, [3])
        check(got, want, dtype, f"long decoding {dtype}")


def planted(cfg, weights, token_a, token_b, strength):
    """Make the key of token `token_a` stand out for queries of token `token_b` in layer 0 (an attention layer that
    leaves some dimensions unrotated): a direction r in the unrotated dimensions of every head is added to the key
    of the normed embedding of a and to the query of that of b, so that their score is about `strength` above the
    others wherever b may see a, and a's value is made large. Neighbours mix in through the convolutions, which
    leaves the planted part in place (the filters' newest tap is near 1)."""
    w = {k: v.clone().float() for k, v in weights.items()}
    m = cfg["layers"][0]["mixer"]
    C, D, E, H, G = cfg["width"], m["dim"], m["vdim"], m["heads"], m["kv_heads"]
    S = cfg.get("streams") or 1
    rot = m["rot"]["dims"] if m.get("rot") else 0
    assert rot < D

    def normed(token):
        u = sum(w["l0.hc1.in"][s] for s in range(S)) * w["embed"][token] if cfg.get("streams") else w["embed"][token]
        return plain.layer_norm(u.double(), w["l0.norm1"].double(), cfg["norm"]["eps"]).float()

    ha, hb = normed(token_a), normed(token_b)
    amount = (strength / float(m["scale"])) ** 0.5
    for g in range(G):
        w["l0.mix.k"][g * D + rot:(g + 1) * D] += amount / (D - rot) ** 0.5 * ha[None, :] / ha.pow(2).sum()
        w["l0.mix.v"][g * E:(g + 1) * E] += 3.0 * ha[None, :] / ha.pow(2).sum()
    for h in range(H):
        w["l0.mix.q"][h * D + rot:(h + 1) * D] += amount / (D - rot) ** 0.5 * hb[None, :] / hb.pow(2).sum()
    return {k: v.to(torch.bfloat16) for k, v in w.items()}


EDGE = mu.make_config([
    mu.attention_layer(heads=2, kv_heads=1, dim=32, vdim=32, conv=3, window=20, rot_dims=16, scale=0.25, ff=48),
    mu.attention_layer(heads=2, kv_heads=1, dim=32, vdim=32, conv=3, window=33, rot_dims=16, scale=0.25, kv_from=0, ff=0),
], vocab=30, width=32, streams=2, taps=2)


def test_window_edges_with_a_planted_key(ops, tmp_path):
    """Token A's key and value stand out for queries of token B. B stands just inside and just outside the windows of
    both layers (20, and 33 on the borrowed keys), behind page borders, in a prompt and in decoding; A also is the very
    first token. A window that is one token off moves the logits there by far more than the tolerance, which the
    plain implementation with a window one longer or shorter shows."""
    A, B = 7, 11
    weights = planted(EDGE, mu.random_weights(EDGE, seed=9, dtype=torch.float32), A, B, strength=30.0)
    folder = mu.write_model(tmp_path / "edge", EDGE, weights)
    filler = [t for t in mu.random_ids(EDGE, 400, seed=2) if t not in (A, B)]
    ids = filler[:75]
    places = {0: A, 19: B, 20: B, 32: B, 33: B, 40: A, 59: B, 60: B, 61: B, 72: B, 73: B, 74: B}
    for at, token in places.items():
        ids[at] = token
    want = mu.oracle(EDGE, weights, ids)
    # the test can see a window that is one token off: in layer 0, where the key is planted, by more than the
    # bfloat16 bound; in the layer that borrows (its queries are not planted), by more than the float32 bound
    for delta, own, borrowed in ((-1, [19, 59], [32, 72]), (1, [20, 60], [33, 73])):
        off = {**EDGE, "layers": [dict(l, mixer={**l["mixer"], "mask": {"size": l["mixer"]["mask"]["size"] + delta}})
                                  for l in EDGE["layers"]]}
        moved = mu.logit_error(mu.oracle(off, weights, ids), want)
        assert float(moved[own].min()) > 2 * mu.TOL[torch.bfloat16]
        assert float(moved[borrowed].max()) > 5 * mu.TOL[torch.float32]
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype)
        check(whole(llm, "a", ids), want, dtype, f"prompt {dtype}")
        check(in_portions(llm, "b", ids, [17, 2, 13]), want, dtype, f"portions, then decoding {dtype}")
        check(in_portions(llm, "c", ids, [58]), want, dtype, f"decoding over the second edge {dtype}")


def test_far_state_reaches_the_present(ops, tmp_path):
    """A state mixer with a slow decay: what the first tokens wrote still shows hundreds of tokens later, through a
    prompt in one piece, in portions and in decoding (the state is carried, not recomputed); a fast head beside it
    forgets. Shown by the plain implementation on the same tokens with another first token."""
    cfg = mu.make_config([mu.lightning_layer(heads=2, dim=16, vdim=16, decay=(0.999, 0.5), ff=0)],
                         vocab=30, width=32, streams=2, taps=0)
    weights = mu.random_weights(cfg, seed=4, dtype=torch.bfloat16)
    ids = mu.random_ids(cfg, 260, seed=8)
    want = mu.oracle(cfg, weights, ids)
    other = mu.oracle(cfg, weights, [(ids[0] + 1) % 30] + ids[1:])
    assert float(mu.logit_error(other[-5:], want[-5:]).min()) > 10 * mu.TOL[torch.float32]
    folder = mu.write_model(tmp_path / "far", cfg, weights)
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype)
        check(whole(llm, "a", ids)[-40:], want[-40:], dtype, f"whole {dtype}")
        check(in_portions(llm, "b", ids, [64, 2, 100, 61])[-40:], want[-40:], dtype, f"portions {dtype}")


def test_greedy_generation_through_the_scheduler(ops, folders):
    """`LLM.generate`: continuous batching with a token budget that cuts the prompts, more requests than seats, and
    (on the GPU) captured decode steps. Every token is the plain implementation's greedy pick given what came before,
    or a near tie."""
    folder, cfg, weights = folders["mixed"]
    prompts = [mu.random_ids(cfg, n, seed=40 + n) for n in (23, 5, 14, 9, 2)]
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype, num_blocks=64, max_seqs=3, token_budget=16,
                     use_graphs=ops.device.type != "cpu")
        outs = llm.generate(prompts, SamplingParams(max_new_tokens=12))
        slack = 1e-3 if dtype == "float32" else 0.35
        for prompt, out in zip(prompts, outs):
            assert len(out.token_ids) == 12
            ids = list(prompt)
            for token in out.token_ids:
                logits = mu.oracle(cfg, weights, ids)[-1]
                assert float(logits[token]) >= float(logits.max()) - slack * float(logits.abs().max()), (dtype, out.token_ids)
                ids.append(token)
        assert not llm.cache.live()
        llm.close()


def test_random_model_folder_reads_back(tmp_path):
    """`random-model` of the command line writes a folder that the loader takes, tensor for tensor as the design
    names them."""
    import json

    from distie_amd import cli
    from distie_amd.weights.safetensors_io import SafetensorsFile

    (tmp_path / "config.json").write_text(json.dumps(PLAIN))
    assert cli.main(["random-model", "--config-json", str(tmp_path / "config.json"), "--out", str(tmp_path / "m"),
                     "--seed", "3", "--dtype", "bf16", "--std", "0.1"]) == 0
    stored = SafetensorsFile(tmp_path / "m" / "model.safetensors")
    assert {name: tuple(entry[1]) for name, entry in stored.index.items()} == mu.tensor_shapes(PLAIN)
    stored.close()
    llm = engine(tmp_path / "m", TorchOps(), "float32")
    assert llm.step([StepEntry("a", [1, 2, 3], [2])]).shape == (1, PLAIN["vocab"])


@pytest.mark.gpu
def test_trace_runner_and_command_line(folders, tmp_path):
    """The trace runner as a program (its own process, steps on standard input, four requests live, pages and
    slots used again) and `generate` of the command line, on a Musutar model, against the plain implementation."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parents[1]
    folder, cfg, weights = folders["mixed"]
    lengths = {"p": 70, "q": 33, "r": 64, "s": 5, "t": 90, "u": 41}
    reqs = {r: mu.random_ids(cfg, n, 60 + n) for r, n in lengths.items()}
    want = {r: mu.oracle(cfg, weights, ids) for r, ids in reqs.items()}
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
            logits = mu.oracle(cfg, weights, ids)[-1]
            assert float(logits[token]) >= float(logits.max()) - 1e-3 * float(logits.abs().max())
            ids.append(token)


def test_preemption_starts_the_state_over(ops, folders):
    """So few pages that running requests are preempted and recomputed: their convolution inputs and decayed
    states start from zero again, and every token still is the plain implementation's pick."""
    folder, cfg, weights = folders["plain"]          # one of its layers keeps every key: the pages grow with the request
    prompts = [mu.random_ids(cfg, n, seed=70 + n) for n in (20, 26, 17)]
    block = 4 if ops.device.type == "cpu" else 16
    new = 24 if block == 4 else 40
    # as many pages as the longest request may hold by itself: three of them do not fit side by side
    llm = engine(folder, ops, "float32", block_size=block, num_blocks=-(-(26 + new) // block) + 1, max_seqs=3, token_budget=32)
    outs = llm.generate(prompts, SamplingParams(max_new_tokens=new))
    assert sum(o.preemptions for o in outs) > 0, "the pool was not small enough to preempt anybody"
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for token in out.token_ids:
            logits = mu.oracle(cfg, weights, ids)[-1]
            assert float(logits[token]) >= float(logits.max()) - 1e-3 * float(logits.abs().max())
            ids.append(token)
    llm.cache.check()
    assert not llm.cache.live()
