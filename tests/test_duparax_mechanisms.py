"""Each mechanism of the Duparax decoder alone, as the kernel surface offers it, against the matching function of
the plain implementation: on the CPU test double and on the GPU kernels (float32 and bfloat16 operands).

A step here is a batch of several requests' rows; states are carried over several steps, with slots that are
taken in any order, and the result must be that of the whole sequence run at once."""

import torch
import pytest

import plain_duparax as plain
from distie_amd.cache import CacheManager
from distie_amd.config.model_config import PartSpec
from distie_amd.engine.batch import BatchBuilder, StepEntry
from distie_amd.parts import FixedState, StepContext, TensorDecl, build_part
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

    def __init__(self, ops, needs, lengths, cuts, block=4, slots=5, dtype=torch.float32):
        self.ops = ops
        self.cache = CacheManager([{"mixer": needs}], block, 64, slots, device=ops.device, dtype=dtype)
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
LONG_LENGTHS = (150, 1, 70, 33)
LONG_CUTS = ((100, 1, 2, 0), (17, 0, 64, 33), (33, 0, 4, 0))


def gather(seqs, rows):
    return torch.cat([seqs[i][at:at + n] for i, at, n in rows])


@pytest.mark.parametrize("width", [30, 40, 48, 256, 2048])
def test_norms_behind_sub_layers_and_normed_sums(ops, width):
    T, C = 7, width
    dev = lambda t: t.to(ops.device)
    wl, wr, post, pre = (1 + rnd(C, seed=s, scale=0.2) for s in (1, 2, 3, 4))
    for dtype in act_types(ops):
        a, b = rnd(T, C, seed=5, scale=3.0).to(dtype), rnd(T, C, seed=6, scale=0.2).to(dtype)
        want_sum = 0.5 * (plain.rms_norm(a.to(F), wl.to(F), 1e-5) + plain.rms_norm(b.to(F), wr.to(F), 1e-5))
        both = ops.normed_sum([dev(a), dev(b)], [dev(wl), dev(wr)], 1e-5, 0.5)
        close(ops.dense(both), want_sum, torch.float32, "normed sum")
        one = ops.normed_sum([dev(b)], [dev(wr)], 1e-5, 1.0)
        close(ops.dense(one), plain.rms_norm(b.to(F), wr.to(F), 1e-5), torch.float32, "one normed term")
        x = rnd(T, C, seed=7)
        residual = dev(x.clone())
        h = ops.add_normed_rmsnorm(residual, both, dev(post), 1e-6, dev(pre), 1e-4, dtype)
        want_x = x.to(F) + plain.rms_norm(want_sum, post.to(F), 1e-6)
        close(residual, want_x, torch.float32, "residual behind the sum")
        close(ops.dense(h), plain.rms_norm(want_x, pre.to(F), 1e-4), dtype, "the next norm")
        ops.add_normed(residual, dev(a), dev(post), 1e-6)
        want_x = want_x + plain.rms_norm(a.to(F), post.to(F), 1e-6)
        close(residual, want_x, torch.float32, "residual behind a plain term")
        # what a product returns, in whatever form, is a term as well
        weight = rnd(C, 24, seed=8, scale=0.3).to(dtype)
        y = rnd(T, 24, seed=9).to(dtype)
        product = ops.linear(dev(y), dev(weight))
        ops.add_normed(residual, product, dev(post), 1e-6)
        rounded = (y.to(F) @ weight.to(F).T).to(dtype).to(F)
        close(residual, want_x + plain.rms_norm(rounded, post.to(F), 1e-6), dtype, "residual behind a product")


@pytest.mark.parametrize("lengths,cuts", [(LENGTHS, CUTS), (LONG_LENGTHS, LONG_CUTS)])
@pytest.mark.parametrize("heads,dim,vdim,tau", [(2, 8, 16, 4.0), (3, 16, 8, 1.0), (1, 32, 32, 16.0), (2, 40, 72, 64.0),
                                                (2, 128, 64, 16.0), (1, 12, 20, 2.0)])
def test_gated_decayed_state(ops, heads, dim, vdim, tau, lengths, cuts):
    """The state with a decay for every key channel and token, handed from step to step; decays from fast to slow.
    The decay's logits are given, or made from a few columns behind q, k and v (inside the scan, for few rows)."""
    rank = 5 if dim == 12 else 8
    first = heads * (2 * dim + vdim)
    width = first + 3 + rank                                   # further columns are left alone; the last are `low`
    up, bias = rnd(heads * dim, rank, seed=3, scale=1.5), rnd(heads * dim, seed=4, scale=2.0) + 2.0
    for dtype in act_types(ops):
        seqs = [rnd(n, width, seed=20 + i).to(dtype) for i, n in enumerate(lengths)]
        logits = [s[:, first + 3:].to(F) @ up.to(dtype).to(F).T + bias.to(F) for s in seqs]
        want = []
        for s, z in zip(seqs, logits):
            s = s.to(F)
            q = s[:, :heads * dim].view(-1, heads, dim) * dim ** -0.5
            k = s[:, heads * dim:2 * heads * dim].view(-1, heads, dim)
            v = s[:, 2 * heads * dim:first].view(-1, heads, vdim)
            alpha = torch.sigmoid(z).pow(1.0 / tau).view(-1, heads, dim)
            want.append(plain.gated_linear_recurrence(q, k, v, alpha).reshape(-1, heads * vdim))
        for given in (True, False):
            steps = Steps(ops, FixedState.of((heads, dim, vdim)), lengths, cuts)
            for meta, rows in steps:
                product = gather(seqs, rows).to(ops.device)
                if given:
                    got = ops.gated_decay_scan(product, gather(logits, rows).float().to(ops.device), steps.view()["state"],
                                               meta, heads, dim, vdim, dim ** -0.5, tau)
                else:
                    low = (product[:, first + 3:], up.to(dtype).to(ops.device), bias.to(ops.device))
                    got = ops.gated_decay_scan(product, None, steps.view()["state"], meta, heads, dim, vdim, dim ** -0.5,
                                               tau, low)
                assert got.dtype == torch.float32
                close(got, gather(want, rows), torch.float32, f"rows {rows}, logits given: {given}")


def test_norm_of_every_head_with_a_silu_gate(ops):
    T, H, E = 6, 3, 24
    for dtype in act_types(ops):
        wide = rnd(T, 16 + H * E, seed=2).to(dtype)
        gates = wide.to(ops.device)[:, 16:]                       # a view with a row stride
        y, weight = rnd(T, H * E, seed=3, scale=3.0), 1 + rnd(E, seed=4, scale=0.2)
        y[:, E:2 * E] *= 50.0                                     # a head's norm must not see its neighbours
        got = ops.rmsnorm_gate(y.to(ops.device), weight.to(ops.device), 1e-5, gates, dtype, group=E, gate="silu")
        want = plain.rms_norm(y.to(F).view(T, H, E), weight.to(F), 1e-5).reshape(T, H * E) * plain.silu(wide.to(F)[:, 16:])
        close(got, want, dtype, "norm per head, silu gate")
        got = ops.rmsnorm_gate(y.to(ops.device), weight.to(ops.device), 1e-5, None, dtype, group=E)
        close(got, plain.rms_norm(y.to(F).view(T, H, E), weight.to(F), 1e-5).reshape(T, H * E), dtype, "norm per head")
        # columns kept out of wider heads, no gate
        x = rnd(T, H * 32, seed=5).to(dtype)
        got = ops.sigmoid_gate(x.to(ops.device), H, 32, E, None)
        close(got, x.to(F).view(T, H, 32)[..., :E].reshape(T, H * E), dtype, "kept columns")


@pytest.mark.parametrize("lengths,cuts", [(LENGTHS, CUTS), (LONG_LENGTHS, LONG_CUTS)])
@pytest.mark.parametrize("width,blocks,taps", [(64, 4, 4), (40, 4, 3), (48, 1, 1), (32, 32, 2), (200, 2, 2)])
def test_recurrent_unit(ops, width, blocks, taps, lengths, cuts, monkeypatch):
    """Convolution with a bias on a view of columns, block-diagonal gates, the recurrence and the product with the
    other branch, with the inputs and the state handed from step to step. Long portions go through the scan in
    chunks of rows (on the GPU)."""
    if hasattr(ops, "LRU_CHUNKED_MIN_ROWS"):
        monkeypatch.setattr(ops, "LRU_CHUNKED_MIN_ROWS", 16)
    R, n = width, width // blocks
    for dtype in act_types(ops):
        conv, conv_b = rnd(R, taps, seed=1, scale=0.5).to(dtype), rnd(R, seed=2, scale=0.3)
        ra, ri = rnd(blocks, n, n, seed=3, scale=1.5 / n ** 0.5).to(dtype), rnd(blocks, n, n, seed=4, scale=1.5 / n ** 0.5).to(dtype)
        ra_b, ri_b, lam = rnd(blocks, n, seed=5, scale=0.5), rnd(blocks, n, seed=6, scale=0.5), rnd(R, seed=7) - 2.0
        seqs = [rnd(length, 2 * R, seed=20 + i).to(dtype) for i, length in enumerate(lengths)]     # y branch, x branch
        want = []
        for s in seqs:
            u = plain.causal_conv(s.to(F)[:, R:], conv.to(F), conv_b.to(F)).to(dtype).to(F)
            r = torch.sigmoid(plain.block_diagonal(u, ra.to(F), ra_b.to(F)))
            i = torch.sigmoid(plain.block_diagonal(u, ri.to(F), ri_b.to(F)))
            want.append(plain.real_gated_recurrence(u, r, i, lam.to(F)) * plain.gelu_tanh(s.to(F)[:, :R]))
        tensors = [TensorDecl("state", (R,), torch.float32)] + ([TensorDecl("conv", (taps - 1, R), torch.float32)] if taps > 1 else [])
        steps = Steps(ops, FixedState(tuple(tensors)), lengths, cuts)
        dev = lambda t: t.to(ops.device)
        for meta, rows in steps:
            product = dev(gather(seqs, rows))
            u = ops.causal_conv(product[:, R:], dev(conv), steps.view()["conv"] if taps > 1 else None, meta, bias=dev(conv_b))
            a, x = ops.lru_gates(u, dev(ra), dev(ra_b), dev(ri), dev(ri_b), dev(lam), 8.0)
            got = ops.lru_scan(a, x, steps.view()["state"], meta, product[:, :R], "gelu_tanh", dtype)
            close(got, gather(want, rows), dtype, f"rows {rows}")


@pytest.mark.parametrize("experts,top,width", [(6, 2, 48), (12, 3, 40), (4, 4, 32), (5, 1, 256), (70, 8, 64)])
def test_router(ops, experts, top, width):
    T = 9
    for dtype in act_types(ops):
        x = rnd(T, width, seed=1).to(dtype)
        weight, bias = rnd(experts, width, seed=2, scale=0.5).to(dtype), rnd(experts, seed=3)
        chosen, gates = ops.route_topk(x.to(ops.device), weight.to(ops.device), bias.to(ops.device), top)
        z = x.to(F) @ weight.to(F).T + bias.to(F)
        best = torch.topk(z, top, dim=-1)
        assert chosen.dtype == torch.int32 and chosen.cpu().tolist() == best.indices.tolist()
        close(gates, torch.softmax(best.values, -1), torch.float32, "weights of the chosen")
        factor = torch.zeros(T, experts, dtype=F).scatter_(1, best.indices, torch.softmax(best.values, -1))
        for more in (5, 16):                                      # columns behind the experts' that every row keeps
            hidden = rnd(T, experts * 8 + more, seed=4).to(dtype)
            got = ops.route_scale(hidden.clone().to(ops.device), chosen, gates, experts, 8)
            want = hidden.to(F).clone()
            want[:, :experts * 8] = (want[:, :experts * 8].view(T, experts, 8) * factor[:, :, None]).view(T, -1)
            close(got, want, dtype, "hidden values of the experts")
    # equal logits: the lower index wins
    same = torch.zeros(2, 16)
    chosen, gates = ops.route_topk(same.to(ops.device), torch.ones(5, 16).to(ops.device), None, 2)
    assert chosen.cpu().tolist() == [[0, 1], [0, 1]] and torch.allclose(gates.cpu(), torch.full((2, 2), 0.5))


@pytest.mark.parametrize("experts,top,ff,shared", [(6, 2, 24, 40), (3, 3, 8, 0), (5, 1, 16, 16)])
def test_routed_feed_forward(ops, experts, top, ff, shared):
    C, T = 48, 11
    spec = PartSpec("routed_experts", "m.", {"hidden_size": C, "num_experts": experts, "top": top, "expert_size": ff,
                                             "shared_size": shared})
    for dtype in act_types(ops):
        part = build_part("feed_forward", spec)
        w = {name: rnd(*s.shape, seed=30 + i, scale=1.0 if name.startswith("router") else 0.3).to(dtype)
             for i, (name, s) in enumerate(part.param_specs().items())}
        part.load({k: v.to(ops.device) for k, v in w.items()})
        x = rnd(T, C, seed=5).to(dtype)
        mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
        if shared:
            mlp["shared"] = {"ff": shared}
        want = plain.routed_mlp(x.to(F), {"m." + k: v.to(F) for k, v in w.items()}, "m.", mlp)
        got = ops.dense(part.forward(ops, x.to(ops.device), StepContext(None, dtype)))
        close(got, want, dtype, "mixture of experts")


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,coef,every,lengths,cuts", [
    (4, 2, 16, 24, 0.7, 5, LENGTHS, CUTS), (2, 2, 32, 32, 1.0, 1, LENGTHS, CUTS), (5, 1, 20, 12, 0.5, 3, LENGTHS, CUTS),
    (3, 1, 40, 16, 0.0, 0, LENGTHS, CUTS), (4, 2, 48, 64, 0.5, 64, LONG_LENGTHS, LONG_CUTS),
    (2, 1, 64, 32, 0.25, 16, LONG_LENGTHS, LONG_CUTS)])
def test_attention_with_biases_and_a_query_temperature(ops, heads, kv_heads, dim, vdim, coef, every, lengths, cuts):
    """The left mixer alone over a batch in steps: biases, the temperature by position (its steps fall inside
    portions, at their starts and on single rows), keys and values of different sizes, no gate and no rotation."""
    C = 48
    temp = {"coef": coef, "every": every} if every else None
    params = {"hidden_size": C, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": dim, "value_dim": vdim,
              "conv_taps": 0, "window": None, "scale": 0.2, "output_gate": False, "bias": True, "position": None,
              "q_temp": temp}
    cfg = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 0.2, "q_temp": temp}
    for dtype in act_types(ops):
        part = build_part("mixer", PartSpec("conv_gated_attention", "a.", params))
        w = {name: rnd(*s.shape, seed=30 + i, scale=0.5 if name.endswith(".b") else 0.25).to(dtype)
             for i, (name, s) in enumerate(part.param_specs().items())}
        part.load({k: v.to(ops.device) for k, v in w.items()})
        seqs = [rnd(n, C, seed=50 + i).to(dtype) for i, n in enumerate(lengths)]
        want = [plain.left_mixer(s.to(F), {"m." + k: v.to(F) for k, v in w.items()}, "m.", cfg) for s in seqs]
        steps = Steps(ops, part.cache_requirement(), lengths, cuts, block=16, dtype=dtype)
        for meta, rows in steps:
            x = gather(seqs, rows).to(ops.device)
            got = ops.dense(part.forward(ops, x, StepContext(meta, dtype), steps.view(), True))
            close(got, gather(want, rows), dtype, f"rows {rows}")
        steps.cache.check()
