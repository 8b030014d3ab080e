"""Each mechanism of the Musutar decoder alone, as the kernel surface offers it, against the matching function of
the plain implementation: on the CPU test double and on the GPU kernels (float32 and bfloat16 operands).

A step here is a batch of several requests' rows; states are carried over several steps, with slots that are
taken in any order, and the result must be that of the whole sequence run at once."""

import math

import torch
import pytest

import plain_musutar as plain
from distie_amd.cache import CacheManager
from distie_amd.config.model_config import PartSpec
from distie_amd.engine.batch import BatchBuilder, StepEntry
from distie_amd.parts import FixedState, TensorDecl, build_part
from torch_ops import TorchOps

F = torch.float64


@pytest.fixture(scope="module", params=["cpu", pytest.param("hip", marks=pytest.mark.gpu)])
def ops(request):
    if request.param == "cpu":
        return TorchOps()
    from distie_amd.kernels.hip_ops import HipOps

    return HipOps("cuda:0")


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def act_types(ops):
    return [torch.float32] if ops.device.type == "cpu" else [torch.float32, torch.bfloat16]


def close(got, want, dtype, what=""):
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    err = (got.double().cpu() - want.double()).abs().max() / (want.double().abs().max() + 1e-9)
    assert float(err) < tol, f"{what}: {float(err)}"


class Steps:
    """Sequences fed in steps through a cache manager: step k brings cuts[k][i] rows of sequence i (0: left out)."""

    def __init__(self, ops, needs, lengths, cuts, block=4, slots=5):
        self.ops = ops
        self.cache = CacheManager([{"mixer": needs}], block, 64, slots, device=ops.device, dtype=torch.float32)
        self.builder = BatchBuilder(self.cache, 512, ops.device, 1000)
        self.lengths, self.cuts = lengths, cuts
        # slots are not taken in the order of the sequences
        for i in reversed(range(len(lengths))):
            self.cache.add(i)
        self.at = [0] * len(lengths)

    def __iter__(self):
        for cut in self.cuts:
            entries, rows = [], []
            for i, n in enumerate(cut):
                n = min(n, self.lengths[i] - self.at[i])
                if n < 1:
                    continue
                self.cache.reserve(i, n)
                entries.append(StepEntry(i, [0] * n, []))
                rows.append((i, self.at[i], n))
            if not entries:
                continue
            _, meta, _ = self.builder.build(entries)
            yield meta, rows
            for i, at, n in rows:
                self.cache.commit(i, n)
                self.at[i] += n
        assert self.at == list(self.lengths), "the cuts do not cover the sequences"

    def view(self):
        return self.cache.layer(0)["mixer"]


LENGTHS = (13, 1, 9, 6)
CUTS = ((5, 1, 2, 0), (1, 0, 1, 6), (2, 0, 0, 0), (1, 0, 6, 0), (4, 0, 0, 0))


def gather(seqs, rows):
    return torch.cat([seqs[i][at:at + n] for i, at, n in rows])


@pytest.mark.parametrize("streams", [1, 2, 4])
@pytest.mark.parametrize("norm", ["layer", "rms", "none"])
def test_streams_step(ops, streams, norm):
    T, C, S = 7, 40, streams
    init, delta, gate = rnd(T, C, seed=1), rnd(T, C, seed=2), rnd(T, C, seed=3)
    mix, write, read = torch.eye(S) + rnd(S, S, seed=4, scale=0.3), 1 + rnd(S, seed=5, scale=0.3), rnd(S, seed=6)
    weight = 1 + rnd(C, seed=7, scale=0.2)
    dev = lambda t: t.to(ops.device)
    for dtype in act_types(ops):
        x, h = ops.hyper_step(None, init=dev(init), read=dev(read), norm_weight=dev(weight), norm=norm, eps=1e-5,
                              out_dtype=dtype)
        want_x = init.to(F)[:, None, :].repeat(1, S, 1)

        def read_of(xs):
            u = torch.einsum("s,tsc->tc", read.to(F), xs)
            if norm == "layer":
                return plain.layer_norm(u, weight.to(F), 1e-5)
            return plain.rms_norm(u, weight.to(F), 1e-5) if norm == "rms" else u

        close(x, want_x, torch.float32, "streams made")
        close(h, read_of(want_x), dtype, "first read")
        d, g = delta.to(dtype), gate.to(dtype)
        _, h = ops.hyper_step(x, delta=dev(d), gate=dev(g), mix=dev(mix), write=dev(write), read=dev(read),
                              norm_weight=dev(weight), norm=norm, eps=1e-5, out_dtype=dtype)
        y = d.to(F) * torch.sigmoid(g.to(F))
        want_x = torch.einsum("sj,tsc->tjc", mix.to(F), want_x) + write.to(F)[None, :, None] * y[:, None, :]
        close(x, want_x, torch.float32, "streams written")
        close(h, read_of(want_x), dtype, "second read")
        # without a gate, and the plain sum at the end
        _, total = ops.hyper_step(x, delta=dev(d), mix=dev(mix), write=dev(write), read=dev(torch.ones(S)))
        want_x = torch.einsum("sj,tsc->tjc", mix.to(F), want_x) + write.to(F)[None, :, None] * d.to(F)[:, None, :]
        close(total, want_x.sum(1), torch.float32, "sum of the streams")
    got = ops.layernorm(dev(init), dev(weight), 1e-5, torch.float32)
    close(got, plain.layer_norm(init.to(F), weight.to(F), 1e-5), torch.float32, "layernorm")


@pytest.mark.parametrize("taps,residual", [(1, True), (2, False), (3, True), (4, False), (7, False)])
def test_convolution_over_time_with_carried_inputs(ops, taps, residual):
    N = 70
    w = rnd(N, taps, seed=1, scale=0.5)
    for dtype in act_types(ops):
        seqs = [rnd(n, N, seed=10 + i).to(dtype) for i, n in enumerate(LENGTHS)]
        want = [plain.causal_conv(s.to(F), w.to(dtype).to(F)) + (s.to(F) if residual else 0) for s in seqs]
        needs = FixedState((TensorDecl("history", (taps - 1, N), torch.float32),)) if taps > 1 else None
        steps = Steps(ops, needs, LENGTHS, CUTS)
        for meta, rows in steps:
            state = steps.view()["history"] if taps > 1 else None
            got = ops.causal_conv(gather(seqs, rows).to(ops.device), w.to(dtype).to(ops.device), state, meta, residual)
            close(got, gather(want, rows), dtype, f"taps {taps} rows {rows}")


LONG_LENGTHS = (150, 1, 70, 33)
LONG_CUTS = ((100, 1, 2, 0), (17, 0, 64, 33), (33, 0, 4, 0))


@pytest.mark.parametrize("lengths,cuts", [(LENGTHS, CUTS), (LONG_LENGTHS, LONG_CUTS)])
@pytest.mark.parametrize("heads,dim,vdim", [(2, 8, 16), (3, 16, 8), (1, 32, 32), (2, 40, 72), (2, 128, 64)])
def test_decayed_state_scan(ops, heads, dim, vdim, lengths, cuts):
    """Short portions go row after row, long ones in chunks of rows worked side by side (on the GPU): the same
    recurrence either way, with the state handed from step to step."""
    decay = torch.tensor([0.999, 0.6, 0.9][:heads], dtype=torch.float32)
    width = heads * (2 * dim + vdim) + 5                       # further columns are left alone
    for dtype in act_types(ops):
        seqs = [rnd(n, width, seed=20 + i).to(dtype) for i, n in enumerate(lengths)]
        want = []
        for s in seqs:
            z = plain.silu(s.to(F))
            q, k = z[:, :heads * dim].view(-1, heads, dim), z[:, heads * dim:2 * heads * dim].view(-1, heads, dim)
            v = z[:, 2 * heads * dim:heads * (2 * dim + vdim)].view(-1, heads, vdim)
            want.append(plain.decayed_state_scan(q, k, v, decay.tolist()).reshape(-1, heads * vdim))
        steps = Steps(ops, FixedState.of((heads, dim, vdim)), lengths, cuts)
        for meta, rows in steps:
            got = ops.decay_scan(gather(seqs, rows).to(ops.device), steps.view()["state"], decay.to(ops.device), meta,
                                 heads, dim, vdim)
            assert got.dtype == torch.float32
            close(got, gather(want, rows), torch.float32 if dtype == torch.float32 else dtype, f"rows {rows}")


def test_gates_norm_and_activations(ops):
    T, H, stride, E = 6, 3, 32, 24
    for dtype in act_types(ops):
        x, wide = rnd(T, H * stride, seed=1).to(dtype), rnd(T, 11 + H * E, seed=2).to(dtype)
        gates = wide.to(ops.device)[:, 11:]                       # a view with a row stride
        got = ops.sigmoid_gate(x.to(ops.device), H, stride, E, gates)
        want = x.to(F).view(T, H, stride)[..., :E].reshape(T, H * E) * torch.sigmoid(wide.to(F)[:, 11:])
        close(got, want, dtype, "sigmoid gate")
        y, weight = rnd(T, H * E, seed=3, scale=3.0), 1 + rnd(H * E, seed=4, scale=0.2)
        got = ops.rmsnorm_gate(y.to(ops.device), weight.to(ops.device), 1e-5, gates, dtype)
        want = plain.rms_norm(y.to(F), weight.to(F), 1e-5) * torch.sigmoid(wide.to(F)[:, 11:])
        close(got, want, dtype, "gated norm")
        z = rnd(T, 50, seed=5, scale=2.0).to(dtype)
        for kind, f in (("relu2", lambda t: torch.relu(t) ** 2), ("silu", plain.silu), ("relu", torch.relu),
                        ("gelu_tanh", lambda t: 0.5 * t * (1 + torch.tanh(math.sqrt(2 / math.pi) * (t + 0.044715 * t ** 3))))):
            close(ops.activation(z.to(ops.device), kind), f(z.to(F)), dtype, kind)


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,rot,taps,window,lends,lengths,cuts", [
    (4, 2, 16, 24, 8, 4, 6, True, LENGTHS, CUTS), (2, 2, 32, 32, 32, 1, None, False, LENGTHS, CUTS),
    (3, 1, 40, 16, 0, 3, 9, False, LENGTHS, CUTS), (2, 1, 16, 16, 16, 0, 4, True, LENGTHS, CUTS),
    (4, 2, 64, 64, 32, 4, 40, True, LONG_LENGTHS, LONG_CUTS), (2, 1, 64, 32, 64, 3, 21, False, LONG_LENGTHS, LONG_CUTS)])
def test_attention_mixer(ops, heads, kv_heads, dim, vdim, rot, taps, window, lends, lengths, cuts):
    """The mixer alone over a batch in steps: projections, convolutions with carried inputs, partial rotation with
    scaled frequencies, the cache write, the window, the output gate; and a second mixer that borrows the first one's
    keys and values with a longer window of its own."""
    C = 48
    position = PartSpec("rope_scaled", "", {"dims": rot, "base": 50.0, "scaling": {
        "factor": 3.0, "original": 16, "fast": 4.0, "slow": 1.0}}) if rot else None
    rot_cfg = {"dims": rot, "base": 50.0, "scaling": {"factor": 3.0, "original": 16, "fast": 4.0, "slow": 1.0}} if rot else None
    longer = None if window is None else window + 3
    params = {"hidden_size": C, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": dim, "value_dim": vdim,
              "conv_taps": taps, "window": window, "keep": longer if lends else window, "scale": 0.2, "position": position}
    for dtype in act_types(ops):
        own = build_part("mixer", PartSpec("conv_gated_attention", "a.", params))
        parts, weights = [own], []
        if lends:
            parts.append(build_part("mixer", PartSpec("conv_gated_attention", "b.", {
                **params, "num_heads": heads * 2, "window": longer, "kv_from": 0})))
        for n, part in enumerate(parts):
            w = {name: rnd(*spec.shape, seed=30 + 7 * n + i, scale=0.5 if name.endswith(".conv") else 0.25).to(dtype)
                 for i, (name, spec) in enumerate(part.param_specs().items())}
            part.load({k: v.to(ops.device) for k, v in w.items()})
            weights.append({"m." + k: v for k, v in w.items()})
        assert "k" not in weights[-1] or not lends
        cache = CacheManager([{"mixer": p.cache_requirement()} for p in parts], 16, 64, 5, device=ops.device, dtype=dtype)
        builder = BatchBuilder(cache, 512, ops.device, 1000)
        seqs = [rnd(n, C, seed=50 + i).to(dtype) for i, n in enumerate(lengths)]
        cfg = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 0.2, "rot": rot_cfg,
               "mask": {"size": window} if window else None}
        want = [[], []]
        for s in seqs:
            pos = torch.arange(s.shape[0])
            y, kv = plain.attention_mixer(s.to(F), {k: v.to(F) for k, v in weights[0].items()}, "m.", cfg, pos)
            want[0].append(y)
            if lends:
                theirs = {**cfg, "heads": heads * 2, "mask": {"size": longer} if longer else None}
                want[1].append(plain.attention_mixer(s.to(F), {k: v.to(F) for k, v in weights[1].items()}, "m.",
                                                     theirs, pos, kv)[0])
        for i in reversed(range(len(lengths))):
            cache.add(i)
        at = [0] * len(lengths)
        from distie_amd.parts import StepContext
        for cut in cuts:
            entries, rows = [], []
            for i, n in enumerate(cut):
                n = min(n, lengths[i] - at[i])
                if n >= 1:
                    cache.reserve(i, n)
                    entries.append(StepEntry(i, [0] * n, []))
                    rows.append((i, at[i], n))
            _, meta, _ = builder.build(entries)
            x = gather(seqs, rows).to(ops.device)
            for n, part in enumerate(parts):
                got = ops.dense(part.forward(ops, x, StepContext(meta, dtype), cache.layer(n)["mixer"], True))
                close(got, gather(want[n], rows), dtype, f"mixer {n} rows {rows}")
            for i, a, n in rows:
                cache.commit(i, n)
                at[i] += n
            cache.check()
