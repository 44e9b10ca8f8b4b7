"""Kisadra on the GPU against the plain implementation (``tests/plain/kisadra_plain.py``): each
mechanism alone (its kernel, and a one-layer model of it), whole prompts, every way of cutting
requests into steps on so few pages and slots that they are used again, keys at the edges of
chunks and pages and far back, and greedy generation through the engine's own entry point."""

from __future__ import annotations

import json
import random
import subprocess
import sys
from pathlib import Path

import pytest
import torch

import kisadra_tiny as kt
import trace_helpers as th
from plain import kisadra_plain as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ROOT = Path(__file__).resolve().parent.parent
#: 32-bit engine against the 32-bit plain implementation, relative to a position's largest logit.
RTOL_F32 = 2e-4
#: bfloat16 engine (weights stored in bfloat16) against the plain implementation in 32-bit on the
#: same weights, for 19 positions in 20; rounding can hand a token to another expert where two
#: router scores are close, so a twentieth of the positions may be off by four times the bound.
RTOL_BF16 = 4e-2
BF16_OUTLIERS = 4.0


@pytest.fixture(scope="module")
def ops():
    from turboserve_amd.kernels.ops import Ops

    return Ops(DEV)


def excess(got: torch.Tensor, want: torch.Tensor, dtype: str) -> float:
    rtol = RTOL_F32 if dtype == "float32" else RTOL_BF16
    bound = rtol * want.abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
    rows = ((got - want).abs() / bound).amax(dim=-1)
    if dtype == "float32":
        return float(rows.max())
    ordered = rows.sort().values
    return max(float(ordered[int(0.95 * (len(ordered) - 1))]), float(ordered[-1]) / BF16_OUTLIERS)


def tokens_of(vocab: int, length: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()


def run_trace(folder, dtype: str, page: int, steps: list[dict], max_tokens: int | None = None, max_live: int = 4):
    from turboserve_amd.engine.replay import TraceReplayer

    replayer = TraceReplayer(folder, dtype=dtype, max_tokens=max_tokens or th.peak_tokens(steps, rounding=page),
                             page_size=page, max_live=max_live)
    outputs = {}
    for record in steps:
        logits = replayer.run_step(record)
        if logits.shape[0]:
            outputs[record["step"]] = logits.float().cpu()
    replayer.manager.check_invariants()
    assert all(pool.num_in_use == 0 for pool in replayer.manager.pools), "pages were not given back"
    assert replayer.manager.state_slots.num_free == max_live, "state slots were not given back"
    return outputs


# ---------------------------------------------------------------------------------------------
# mechanisms alone: kernels
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("inter", [5, 44, 96])
def test_the_tanh_gelu_gated_unit(ops, dtype, inter):
    from turboserve_amd.kernels.ops import GELU_TANH_RULE

    g = torch.Generator().manual_seed(inter)
    gate, up = (3 * torch.randn(9, inter, generator=g)).to(dtype), (3 * torch.randn(9, inter, generator=g)).to(dtype)
    gate[0, 0], gate[0, 1] = -40.0, 40.0  # far out: the sigmoid form must not overflow into NaN
    want = plain.gelu_tanh(gate.float()) * up.float()
    paired = torch.stack([gate, up], dim=2).reshape(9, 2 * inter).contiguous()
    got = ops.swiglu(paired.to(DEV), paired=True, rule=GELU_TANH_RULE).float().cpu()
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got, want, **tol)


@pytest.mark.parametrize("outputs,top", [(7, 2), (3, 3), (5, 1), (16, 4), (70, 6)])
def test_the_softmax_router_with_a_correction(ops, outputs, top):
    """Chosen by score plus correction, weighted by the score alone, nothing normalised; the
    correction is made large enough to change who is taken."""
    g = torch.Generator().manual_seed(outputs * 10 + top)
    x = torch.randn(33, 24, generator=g)
    router = 0.5 * torch.randn(outputs, 24, generator=g)
    correction = 0.2 * torch.randn(outputs, generator=g)
    taken, weights = plain.routing(x, router, correction, top)
    plain_taken, _ = plain.routing(x, router, torch.zeros(outputs), top)
    assert not torch.equal(taken, plain_taken), "the correction changes nobody's experts: the test has no teeth"
    got_taken, got_weights, gate = ops.moe_route(x.to(DEV), router.to(DEV), top=top, groups=1, keep=1, scale=1.0,
                                                 softmax=True, correction=correction.to(DEV), normalise=False)
    assert gate is None
    assert torch.equal(got_taken.cpu().long(), taken)
    torch.testing.assert_close(got_weights.cpu(), weights, rtol=1e-5, atol=1e-6)
    if top < outputs:
        assert float(got_weights.sum(dim=1).max()) < 1.0  # not normalised


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_identity_experts_pass_the_token_itself(ops, dtype):
    g = torch.Generator().manual_seed(5)
    tokens, top, hidden, experts = 6, 3, 20, 4
    rows = torch.randn(tokens, hidden, generator=g).to(dtype)
    pair_out = torch.randn(tokens * top, hidden, generator=g)
    weights = torch.rand(tokens, top, generator=g)
    taken = torch.randint(0, experts + 2, (tokens, top), generator=g).to(torch.int32)
    taken[0] = torch.tensor([experts, experts + 1, 0])
    poisoned = pair_out.clone()
    poisoned[(taken >= experts).reshape(-1)] = float("nan")  # what the products leave for an identity pair is not read
    got = ops.moe_combine(poisoned.to(DEV), weights.to(DEV), None, None, dtype, taken=taken.to(DEV), experts=experts,
                          rows=rows.to(DEV))[0].cpu()
    per_pair = torch.where((taken >= experts)[..., None], rows.float()[:, None, :], pair_out.view(tokens, top, hidden))
    torch.testing.assert_close(got, (weights[..., None] * per_pair).sum(dim=1), rtol=1e-5, atol=1e-5)


def test_the_stream_through_the_entering_matrix(ops):
    g = torch.Generator().manual_seed(8)
    x, origin = torch.randn(7, 20, generator=g), torch.randn(7, 20, generator=g)
    pair = ops.stream_pair(x.to(DEV), origin.to(DEV), torch.float32).cpu()
    torch.testing.assert_close(pair, torch.cat([x, origin], dim=1), rtol=0, atol=0)
    stream = x.clone().to(DEV)
    sums = torch.randn(3, 7, 20, generator=g)
    ops.stream_fold(stream, sums.to(DEV), torch.float32)
    torch.testing.assert_close(stream.cpu(), x + sums.sum(0), rtol=0, atol=1e-5)
    ops.stream_fold(stream, origin.to(torch.bfloat16).to(DEV), torch.bfloat16, assign=True)
    torch.testing.assert_close(stream.cpu(), origin.to(torch.bfloat16).float(), rtol=0, atol=0)


@pytest.mark.parametrize("heads,dim,vdim,low,lengths", [
    (2, 16, 24, 8, [1, 5, 70]), (1, 20, 70, 3, [130, 1, 1, 64]), (3, 64, 32, 16, [200, 65]), (2, 130, 8, 1, [9, 129])])
def test_the_state_walk_whole_and_in_pieces(ops, heads, dim, vdim, low, lengths):
    """The recurrence's kernel alone against the token-by-token definition: requests walked whole,
    and cut into pieces that run side by side; a state that is carried over from before."""
    g = torch.Generator().manual_seed(dim + vdim)
    total = sum(lengths)
    key, val = heads * dim, heads * vdim
    proj = torch.randn(total, 2 * key + 2 * val + low, generator=g)
    proj[:, : 2 * key] *= 0.5
    a2, bias = 0.6 * torch.randn(key, low, generator=g), 1.0 + torch.randn(key, generator=g)
    tau = 3.0
    before = 0.3 * torch.randn(len(lengths) + 2, heads, dim, vdim, generator=g)
    slots = torch.tensor([len(lengths) - i for i in range(len(lengths))], dtype=torch.int32)  # not in row order
    want_o = torch.zeros(total, val)
    want_state = before.clone()
    row = 0
    for r, n in enumerate(lengths):
        state = before[slots[r]].clone().double()
        for t in range(row, row + n):
            q = proj[t, :key].view(heads, dim).double() * dim ** -0.5
            k = proj[t, key:2 * key].view(heads, dim).double()
            v = proj[t, 2 * key:2 * key + val].view(heads, vdim).double()
            z = (a2.double() @ proj[t, 2 * key + 2 * val:].double() + bias.double()).view(heads, dim)
            decay = torch.sigmoid(z) ** (1.0 / tau)
            state = decay[..., None] * state + k[..., None] * v[:, None, :]
            want_o[t] = torch.einsum("hdv,hd->hv", state, q).reshape(-1).float()
        want_state[slots[r]] = state.float()
        row += n
    starts = torch.tensor([0, *torch.tensor(lengths).cumsum(0).tolist()], dtype=torch.int32)
    for pieces in (None, 64, 7):
        state = before.clone().to(DEV)
        out = torch.full((total, val), float("nan"), device=DEV)
        plan = None
        if pieces is not None:
            made, carries = ops.linear_state_pieces(lengths, pieces)
            plan = (torch.tensor(made, dtype=torch.int32, device=DEV), torch.tensor(carries, dtype=torch.int32, device=DEV),
                    len(made), len(carries))
        ops.linear_state(proj.to(DEV), a2.to(DEV), bias.to(DEV), tau, state, slots.to(DEV), starts.to(DEV), tokens=total,
                         first_seq=0, num_seqs=len(lengths), heads=heads, head_dim=dim, value_dim=vdim, dtype=torch.float32,
                         out=out, plan=plan)
        torch.testing.assert_close(out.cpu(), want_o, rtol=2e-4, atol=2e-4)
        torch.testing.assert_close(state.cpu(), want_state, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,in_keys,page,rule", [
    (4, 2, 16, 8, False, 16, dict(chunk=20, sinks=1.0, slopes=True)),
    (6, 2, 32, 32, False, 32, dict(chunk=64, sinks=1.0, slopes=True)),
    (16, 1, 80, 64, True, 16, dict()),
    (8, 1, 320, 256, True, 16, dict()),
    (4, 1, 448, 384, True, 16, dict()),
    (70, 1, 40, 24, True, 8, dict(window=33)),
    (8, 4, 128, 128, False, 16, dict(chunk=1024, sinks=2.0, slopes=True, softcap=5.0)),
    (2, 2, 48, 104, False, 64, dict(window=100, sinks=0.5)),
    (2, 1, 64, 256, False, 16, dict(chunk=300)),
    (3, 3, 256, 128, False, 16, dict(sinks=1.0, slopes=True)),
    (2, 1, 256, 256, True, 32, dict(chunk=77)),
    (2, 2, 384, 200, False, 8, dict(slopes=True)),
])
def test_the_tiled_attention_kernel_against_the_generic_one(ops, heads, kv_heads, dim, vdim, in_keys, page, rule):
    """bfloat16 on the matrix cores against the one-wavefront-per-row kernel on the same pages: prompt
    portions that start in the middle of a request, beside single tokens whose keys are shared out over
    several workgroups; every score rule; values in pages of their own or inside the key rows."""
    g = torch.Generator().manual_seed(heads * 100 + dim)
    query_lens = [130, 64, 3, 1, 1, 1]
    contexts = [400, 64, 1100, 1500, 1, 65]
    pages_of = [-(-c // page) for c in contexts]
    total_pages = sum(pages_of) + 3
    order = torch.randperm(total_pages, generator=g).tolist()
    table = torch.zeros((len(contexts), max(pages_of)), dtype=torch.int32)
    for s, n in enumerate(pages_of):
        table[s, :n] = torch.tensor([order.pop() for _ in range(n)])
    k_pages = torch.randn(total_pages, kv_heads, page, dim, generator=g).to(torch.bfloat16)
    v_pages = None if in_keys else torch.randn(total_pages, kv_heads, vdim, page, generator=g).to(torch.bfloat16)
    tokens = sum(query_lens)
    q = (0.5 * torch.randn(tokens, heads * dim, generator=g)).to(torch.bfloat16)
    starts = torch.tensor([0, *torch.tensor(query_lens).cumsum(0).tolist()], dtype=torch.int32)
    token_seq = torch.repeat_interleave(torch.arange(len(query_lens)), torch.tensor(query_lens)).to(torch.int32)
    positions = torch.cat([torch.arange(c - n, c) for c, n in zip(contexts, query_lens)]).to(torch.int32)
    slopes = torch.tensor(plain.distance_slopes(heads), dtype=torch.float32, device=DEV) if rule.get("slopes") else None
    scale = dim ** -0.5
    dev = lambda t: None if t is None else t.to(DEV)
    want = ops.paged_attention_generic(dev(q), heads * dim, dev(k_pages), dev(v_pages), dev(table), dev(token_seq), dev(positions),
                                       heads, scale, rule.get("window"), slopes, rule.get("softcap", 0.0), chunk=rule.get("chunk"),
                                       sinks=rule.get("sinks", 0.0), value_dim=vdim if in_keys else None).float().cpu()
    tiles = torch.tensor(ops.attention_tile_list(query_lens[:3]), dtype=torch.int32, device=DEV)
    got = ops.attention_tiles(dev(q), heads * dim, dev(k_pages), dev(v_pages), dev(table), dev(starts),
                              torch.tensor(contexts, dtype=torch.int32, device=DEV), tokens=tokens, heads=heads, scale=scale,
                              prefill_tiles=tiles, num_prefill_seqs=3, num_decode_seqs=3, max_decode_context=1536,
                              window=rule.get("window"), chunk=rule.get("chunk"), sinks=rule.get("sinks", 0.0), slopes=slopes,
                              softcap=rule.get("softcap", 0.0), value_dim=vdim if in_keys else None).float().cpu()
    assert torch.isfinite(got).all()
    # Both round probabilities' products differently (bfloat16 probabilities here); outputs are averages of values of size one.
    torch.testing.assert_close(got, want, rtol=2e-2, atol=2e-2)


# ---------------------------------------------------------------------------------------------
# mechanisms alone: one-layer models
# ---------------------------------------------------------------------------------------------

ALONE = {
    "chunks": kt.layer(kt.attention(4, 2, 16, 24, 13, scale=0.4), None),
    "chunks_one_head": kt.layer(kt.attention(1, 1, 20, 6, 1), None),
    "latent": kt.layer(kt.latent(3, 16, 8, 12, 24, base=100.0), None),
    "latent_part_turned": kt.layer(kt.latent(2, 8, 12, 20, 9, turned=6, base=7.0, scale=0.6), None),
    "state": kt.layer(kt.gla(2, 16, 24, 4.0, 8), None),
    "state_wide": kt.layer(kt.gla(1, 100, 70, 16.0, 5), None),
    "dense": kt.layer(kt.gla(1, 8, 8, 2.0, 2), kt.dense(44)),
    "routed": kt.layer(kt.gla(1, 8, 8, 2.0, 2), kt.moe(6, 2, 3, 28, 0.8)),
    "routed_all_identity_taken": kt.layer(kt.gla(1, 8, 8, 2.0, 2), kt.moe(1, 3, 4, 12, 2.0)),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", sorted(ALONE))
@pytest.mark.parametrize("looped", [False, True])
def test_one_layer_models(tmp_path, which, dtype, looped):
    """A model of one layer (with and without the entering matrix in front of it): whole, token by
    token from the start, and in portions, against the plain implementation."""
    config = {"architecture": "Kisadra", "vocab": 61, "width": 40, "norm": {"eps": 1e-5}, "layers": [ALONE[which]],
              "loop": {"start": 0, "stop": 1 if looped else 0, "times": 2 if looped else 1}}
    stored = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = kt.make_model_dir(tmp_path / "m", config, 31, stored, std=0.2 if dtype == "float32" else 0.1)
    requests = {"a": tokens_of(61, 75, 1), "b": tokens_of(61, 3, 2)}
    want = {rid: kt.plain_logits(folder, tokens) for rid, tokens in requests.items()}
    for steps in (th.whole(requests), th.prefix_then_single(requests, tail=74), th.portions(requests, (2, 5, 31, 3))):
        got = th.collect(steps, run_trace(folder, dtype, 8, steps), requests)
        for rid in requests:
            assert excess(got[rid], want[rid], dtype) <= 1.0, (which, rid)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_chunked_layer_on_a_pool_smaller_than_the_request(tmp_path, dtype):
    """Layers that read only their own chunk give the pages below it back while the request runs: 150
    tokens go through a pool of 64, in portions and token by token, and every position is still right."""
    chunked = kt.layer(kt.attention(4, 2, 16, 16, 16, scale=0.4), kt.dense(44))
    config = {"architecture": "Kisadra", "vocab": 61, "width": 40, "norm": {"eps": 1e-5}, "layers": [chunked, chunked],
              "loop": {"start": 0, "stop": 1, "times": 2}}
    stored = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = kt.make_model_dir(tmp_path / "m", config, 77, stored, std=0.2 if dtype == "float32" else 0.1)
    requests = {"long": tokens_of(61, 150, 9)}
    want = kt.plain_logits(folder, requests["long"])
    for steps in (th.portions(requests, (20, 3, 11, 2)), th.prefix_then_single(requests, tail=130)):
        got = th.collect(steps, run_trace(folder, dtype, 8, steps, max_tokens=64), requests)["long"]
        assert excess(got, want, dtype) <= 1.0


# ---------------------------------------------------------------------------------------------
# whole models, every cutting
# ---------------------------------------------------------------------------------------------


@pytest.fixture(scope="module", params=sorted(kt.TINY))
def case(request, tmp_path_factory):
    config, seed, page = kt.TINY[request.param]
    base = tmp_path_factory.mktemp(f"kisadra_{request.param}")
    # The folder's own file does not name the decay input's width: it comes from the tensors.
    folders = {"float32": kt.make_model_dir(base / "f32", config, seed, torch.float32, std=0.15),
               "bfloat16": kt.make_model_dir(base / "bf16", config, seed, torch.bfloat16, std=0.08)}
    for folder in folders.values():
        (folder / "config.json").write_text(json.dumps(kt.without_ranks(config)))
    lengths = (1, 2, 37, 150, 70, 9)
    requests = {f"r{i}": tokens_of(config["vocab"], n, 100 * seed + i) for i, n in enumerate(lengths)}
    expected = {dtype: {rid: kt.plain_logits(folder, tokens) for rid, tokens in requests.items()} for dtype, folder in folders.items()}
    return {"name": request.param, "page": page, "folders": folders, "requests": requests, "expected": expected}


def check_against_plain(case, dtype: str, steps: list[dict], **more) -> None:
    outputs = run_trace(case["folders"][dtype], dtype, case["page"], steps, **more)
    got = th.collect(steps, outputs, case["requests"])
    for rid, want in case["expected"][dtype].items():
        worst = excess(got[rid], want, dtype)
        assert worst <= 1.0, f"{case['name']} {dtype} {rid}: {worst:.2f} times the bound"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts(case, dtype):
    check_against_plain(case, dtype, th.whole(case["requests"]))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prefix_then_token_by_token(case, dtype):
    check_against_plain(case, dtype, th.prefix_then_single(case["requests"], tail=40))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(2, 3, 5, 2, 16, 7), (33, 2, 70, 64), (1, 2)])
def test_portions_of_changing_size(case, dtype, sizes):
    check_against_plain(case, dtype, th.portions(case["requests"], sizes))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_on_pages_and_slots_that_are_used_again(case, dtype):
    """Three requests live at a time out of six, on three state slots and a pool sized for the peak:
    every slot and page serves several requests, and a state left by one must not reach the next."""
    steps = th.mixed(case["requests"], (7, 2, 19, 66, 3), max_live=3, decode_tail=9)
    check_against_plain(case, dtype, steps, max_live=3)


def test_long_decoding(case):
    """One short prompt, then 150 tokens one by one (recorded steps), in 32-bit."""
    config = kt.TINY[case["name"]][0]
    tokens = tokens_of(config["vocab"], 156, 4242)
    requests = {"long": tokens}
    steps = th.prefix_then_single(requests, tail=150)
    got = th.collect(steps, run_trace(case["folders"]["float32"], "float32", case["page"], steps), requests)["long"]
    assert excess(got, kt.plain_logits(case["folders"]["float32"], tokens), "float32") <= 1.0, case["name"]


def test_cuttings_agree_in_32_bit(case):
    """The logits of a position do not depend on how its request was cut or batched, beyond rounding."""
    folder, page = case["folders"]["float32"], case["page"]
    ways = {"whole": th.whole(case["requests"]), "single": th.prefix_then_single(case["requests"], tail=40),
            "portions": th.portions(case["requests"], (2, 5, 3, 24)), "mixed": th.mixed(case["requests"], (5, 2, 21, 80), max_live=4)}
    results = {name: th.collect(steps, run_trace(folder, "float32", page, steps), case["requests"]) for name, steps in ways.items()}
    for name, got in results.items():
        for rid, base in results["whole"].items():
            scale = base.abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
            assert float(((got[rid] - base).abs() / scale).max()) <= 5e-5, (name, rid)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_replay_program(case, dtype, tmp_path):
    """``bin/trace_run`` itself on a model folder of this design, steps that want nothing included."""
    if case["name"] != "A":
        pytest.skip("one configuration is enough for the subprocess test")
    steps = th.mixed(case["requests"], (7, 2, 19, 66, 3), max_live=3, decode_tail=9)
    for record in steps[1::3]:
        for entry in record["entries"]:
            entry["want"] = []
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(case["folders"][dtype]), "--dtype", dtype,
         "--out", str(out), "--max-tokens", str(th.peak_tokens(steps)), "--page-size", str(case["page"])],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [line for line in proc.stdout.splitlines() if line.startswith("done ")] == [f"done {s['step']}" for s in steps]
    import numpy as np

    vocab = kt.TINY["A"][0]["vocab"]
    position = {rid: 0 for rid in case["requests"]}
    for record in steps:
        wanted = sum(len(e["want"]) for e in record["entries"])
        path = out / f"{record['step']}.f32"
        assert path.exists() == bool(wanted)
        got = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(wanted, vocab).copy()) if wanted else None
        row = 0
        for entry in record["entries"]:
            for place in entry["want"]:
                want = case["expected"][dtype][entry["id"]][position[entry["id"]] + place]
                assert excess(got[row:row + 1], want[None], dtype) <= (1.0 if dtype == "float32" else BF16_OUTLIERS)
                row += 1
            position[entry["id"]] += len(entry["tokens"])


def random_config(rng: random.Random) -> dict:
    width = rng.choice([40, 52, 64, 72, 96, 100, 128])
    layers = []
    for _ in range(rng.randint(1, 4)):
        kind = rng.choice(["attention", "latent", "gla"])
        if kind == "attention":
            kv = rng.choice([1, 1, 2, 3])
            dim = rng.choice([8, 12, 16, 20, 32, 48])
            mixer = kt.attention(kv * rng.choice([1, 2, 4]), kv, dim, rng.choice([dim, 8, 24, 40]),
                                 rng.choice([1, 2, 5, 16, 33, 64, 500]), scale=rng.choice([dim ** -0.5, 0.2, 0.5]))
        elif kind == "latent":
            rot = rng.choice([2, 4, 8, 16])
            mixer = kt.latent(rng.choice([1, 2, 3, 5]), rng.choice([4, 8, 12, 32]), rot, rng.choice([4, 8, 20, 32]),
                              rng.choice([3, 8, 16, 40]), turned=rng.choice([rot, 2]), base=rng.choice([10.0, 1000.0, 50000.0]))
        else:
            mixer = kt.gla(rng.choice([1, 2, 3]), rng.choice([4, 12, 16, 32, 72]), rng.choice([8, 16, 64, 80]),
                           rng.choice([1.0, 4.0, 16.0]), rng.choice([1, 4, 16]))
        mlp = rng.choice(["dense", "moe", "moe", "none"])
        if mlp == "dense":
            mlp = kt.dense(rng.choice([24, 44, 64, 100]))
        elif mlp == "moe":
            experts, identity = rng.choice([1, 2, 5, 8]), rng.choice([0, 0, 1, 3])
            mlp = kt.moe(experts, identity, rng.randint(1, min(experts + identity, 4)), rng.choice([16, 28, 40]), rng.choice([0.5, 2.0, 7.0]))
        else:
            mlp = None
        layers.append(kt.layer(mixer, mlp))
    start = rng.randint(0, len(layers))
    return {"architecture": "Kisadra", "vocab": rng.choice([50, 97, 256]), "width": width,
            "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers,
            "loop": {"start": start, "stop": rng.randint(start, len(layers)), "times": rng.randint(1, 3)}}


@pytest.mark.parametrize("trial", range(10))
def test_random_configurations_replay_like_plain(trial, tmp_path):
    """Seeded random configurations: one to four layers of any mixers in any order, loops that are
    empty, whole or partial, chunks from one position to longer than any request, identity
    experts or none; whole, token by token and mixed; 32-bit (every position inside the bound)
    and bfloat16 (nine positions in ten)."""
    rng = random.Random(9000 + trial)
    config = random_config(rng)
    lengths = [rng.randint(1, 6), rng.randint(10, 60), rng.randint(100, 200), rng.randint(20, 90)]
    requests = {f"r{i}": [rng.randrange(config["vocab"]) for _ in range(n)] for i, n in enumerate(lengths)}
    for dtype, stored, std in (("float32", torch.float32, 0.15), ("bfloat16", torch.bfloat16, 0.06)):
        folder = kt.make_model_dir(tmp_path / dtype, config, trial, stored, std=std)
        want = {rid: kt.plain_logits(folder, tokens) for rid, tokens in requests.items()}
        ways = (th.whole(requests), th.prefix_then_single(requests, tail=20),
                th.mixed(requests, (7, 2, 40, 150, 3), max_live=4, decode_tail=5))
        for steps in ways:
            outputs = run_trace(folder, dtype, 16, steps, max_tokens=th.peak_tokens(steps))
            got = th.collect(steps, outputs, requests)
            for rid in requests:
                if dtype == "float32":
                    assert excess(got[rid], want[rid], dtype) <= 1.0, (trial, rid, config)
                else:
                    bound = RTOL_BF16 * want[rid].abs().amax(dim=-1).clamp_min(1.0)
                    rows = (got[rid] - want[rid]).abs().amax(dim=-1) / bound
                    assert float(rows.sort().values[int(0.9 * (len(rows) - 1))]) <= 1.0, (trial, rid, config)


# ---------------------------------------------------------------------------------------------
# one key that a query rests on: far back, at page borders, just inside and outside a chunk
# ---------------------------------------------------------------------------------------------

MARK, ASKS = 7, 9  # the token that is looked for and the token whose query looks for it
CHUNK = 40


def marked_config(kind: str) -> dict:
    first = {"chunks": kt.layer(kt.attention(2, 1, 32, 32, CHUNK, scale=0.8), None),
             "latent": kt.layer(kt.latent(2, 32, 8, 32, 32, scale=0.8), None),
             "state": kt.layer(kt.gla(2, 32, 32, 64.0, 4), None)}[kind]
    return {"architecture": "Kisadra", "vocab": 64, "width": 64, "norm": {"eps": 1e-6},
            "layers": [first, kt.layer(kt.gla(1, 8, 8, 2.0, 2), kt.dense(64))], "loop": {"start": 1, "stop": 1, "times": 1}}


def marked_model(folder, kind: str, dtype: torch.dtype):
    """Weights under which the query of token ASKS rests on the key of token MARK wherever that
    lies, and under which what it finds there matters: the first half of the width is what the
    first layer's queries and keys are made of (by one and the same matrix), and there both
    tokens' rows of the table hold the same large vector; the second half is what its values are
    made of, and there only MARK's row is large."""
    config = marked_config(kind)
    tensors = kt.draw_tensors(config, 21, torch.float32, 0.12)
    g = torch.Generator().manual_seed(3)
    address, content = torch.randn(32, generator=g), torch.randn(32, generator=g)
    if kind != "chunks":
        tensors["embed"][:, :32] *= 0.05  # every other token's key is small: the marked one stands out among hundreds
    tensors["embed"][MARK] = torch.cat([5.0 * address, 5.0 * content])
    asking = torch.randn(32, generator=g)  # the latent layer's queries are made from an address of their own
    if kind == "latent":
        tensors["embed"][ASKS] = torch.cat([5.0 * asking, 5.0 * torch.randn(32, generator=g)])
    else:
        tensors["embed"][ASKS] = torch.cat([5.0 * address, 0.2 * tensors["embed"][ASKS][32:]])
    tensors["l0.norm1"].fill_(1.0)
    tensors["l0.mix.o"] *= 10.0
    if kind == "chunks":
        tensors["l0.mix.q"][:, 32:] = 0
        tensors["l0.mix.k"] = tensors["l0.mix.q"][:32].clone()
        tensors["l0.mix.k.norm"] = tensors["l0.mix.q.norm"][:32].clone()
        tensors["l0.mix.v"][:, :32] = 0
        tensors["l0.mix.v"] *= 4.0
    elif kind == "latent":
        # One latent serves keys and values: it holds the address in its first half and the
        # content in its second (16 + 16 of 32); keys read the first, values the second.  The
        # query matrix first turns the asking token's own address into the marked token's and then
        # does what the latent's first half does, so the asking token finds the mark and not itself.
        down = tensors["l0.mix.dkv"]
        down[:16, 32:] = 0
        down[16:32, :32] = 0
        down[:32] *= 3.0
        up_k = torch.zeros(2, 32, 32)
        up_k[:, :16, :16] = torch.eye(16)
        tensors["l0.mix.uk"] = up_k.reshape(64, 32)
        up_v = torch.zeros(2, 32, 32)
        up_v[:, :16, 16:] = 4.0 * torch.randn(16, 16, generator=g)
        tensors["l0.mix.uv"] = up_v.reshape(64, 32)
        query = torch.zeros(2, 40, 64)
        query[:, :16, :32] = 3.0 * down[:16, :32] @ (address[:, None] * asking[None, :] / (asking @ asking))
        tensors["l0.mix.q"] = query.reshape(80, 64)
        tensors["l0.mix.dkv.norm"].fill_(1.0)
    else:
        tensors["l0.mix.q"][:, 32:] = 0
        tensors["l0.mix.k"] = 0.3 * tensors["l0.mix.q"].clone()
        tensors["l0.mix.v"][:, :32] = 0
        tensors["l0.mix.a2.b"].fill_(6.0)  # decays close to one: the state remembers hundreds of tokens
        tensors["l0.mix.a2"] *= 0.1
    tensors = {name: t.to(dtype).contiguous() for name, t in tensors.items()}
    return kt.make_model_dir(folder, config, 0, tensors=tensors)


def marked_case(folder, mark_at: int, length: int):
    """``(tokens, plain logits, how far the last position's logits move without the mark)``."""
    config, tensors = kt.read_model_dir(folder)
    filler = [t for t in tokens_of(64, 2 * length, 77) if t not in (MARK, ASKS)][:length]
    tokens = list(filler)
    tokens[mark_at] = MARK
    tokens[-1] = ASKS
    want = plain.forward(config, tensors, tokens)
    without = list(tokens)
    without[mark_at] = filler[mark_at]
    moved = (plain.forward(config, tensors, without)[-1] - want[-1]).abs().max() / want[-1].abs().max()
    return tokens, want, float(moved)


def check_marked(folder, dtype, tokens, want, places=1):
    requests = {"m": tokens}
    for steps in (th.whole(requests), th.prefix_then_single(requests, tail=30), th.portions(requests, (17, 2, 64, 5))):
        got = th.collect(steps, run_trace(folder, dtype, 16, steps), requests)["m"]
        assert excess(got[-places:], want[-places:], dtype) <= 1.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["latent", "state"])
@pytest.mark.parametrize("mark_at", [0, 1, 15, 16, 17, 128, 250])
def test_a_key_far_back_is_found(tmp_path, kind, dtype, mark_at):
    folder = marked_model(tmp_path / "far", kind, torch.float32 if dtype == "float32" else torch.bfloat16)
    tokens, want, moved = marked_case(folder, mark_at, 300)
    assert moved > 0.2, f"the far key does not matter enough to this model's last logits ({moved:.3f})"
    check_marked(folder, dtype, tokens, want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("length", [3 * CHUNK + 9, 3 * CHUNK + 1, 3 * CHUNK])
@pytest.mark.parametrize("back", [0, 1, 2])
def test_keys_at_a_chunks_edge(tmp_path, dtype, length, back):
    """The asking token sits 8 positions into its chunk, at its first position, or at its last; the
    mark lies at the chunk's first position (seen), or one or two before it (not seen: there the
    logits must not move at all, and a kernel that saw it would move them by much)."""
    folder = marked_model(tmp_path / "edge", "chunks", torch.float32 if dtype == "float32" else torch.bfloat16)
    last = length - 1
    first_of_chunk = (last // CHUNK) * CHUNK
    if first_of_chunk == last and back == 0:
        pytest.skip("the asking token is the chunk's first: the mark cannot share its place")
    mark_at = first_of_chunk - back
    tokens, want, moved = marked_case(folder, mark_at, length)
    if back == 0:
        assert moved > 0.2, f"the key inside the chunk does not matter enough ({moved:.3f})"
    else:
        # (Not nothing: the second layer's state carries a little of every token.  A kernel that let the
        # first layer see this key would move the logits as the key inside the chunk does.)
        assert moved < 0.05, f"a key outside the chunk moves the plain implementation's logits ({moved:.3f})"
    check_marked(folder, dtype, tokens, want, places=3)


# ---------------------------------------------------------------------------------------------
# generation through the engine
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_engine(tmp_path, name):
    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine
    from turboserve_amd.sampling.params import SamplingParams

    config, seed, page = kt.TINY[name]
    folder = kt.make_model_dir(tmp_path / "gen", config, seed + 5, torch.float32, std=0.2)
    raw, tensors = kt.read_model_dir(folder)
    prompts = [tokens_of(config["vocab"], n, 900 + n) for n in (3, 21, 1, 50)]
    new = 40
    want = [kt.greedy(raw, tensors, prompt, new) for prompt in prompts]
    engine = LLMEngine(EngineConfig(
        model=str(folder), dtype="float32",
        scheduler=SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=64, block_size=page, num_blocks=40),
    ))
    outputs = engine.generate(prompts, SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True))
    assert [out.new_token_ids for out in outputs] == want
    # Once more on the same engine: the pages and state slots of the first run are used again.
    again = engine.generate(list(reversed(prompts)), SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True))
    assert [out.new_token_ids for out in again] == list(reversed(want))


def test_the_command_line_serves_the_design(tmp_path, capsys):
    """``engine random-model`` writes a folder from a config.json of the design, ``engine generate``
    completes prompts given as token ids with the plain implementation's greedy tokens, and
    ``engine kv-size`` sizes a cache with one group per distinct page geometry."""
    import re

    from turboserve_amd import cli

    config, _, page = kt.TINY["A"]
    source = tmp_path / "config.json"
    source.write_text(json.dumps(config))
    folder = tmp_path / "model"
    assert cli.main(["engine", "random-model", "--config", str(source), "--out", str(folder), "--seed", "4", "--dtype", "float32"]) == 0
    raw, tensors = kt.read_model_dir(folder)
    prompts = [tokens_of(config["vocab"], n, 600 + n) for n in (4, 19)]
    capsys.readouterr()
    args = ["engine", "generate", "--model", str(folder), "--dtype", "float32", "--max-tokens", "12", "--ignore-eos",
            "--num-blocks", "24", "--block-size", str(page)]
    assert cli.main(args + [a for p in prompts for a in ("--prompt-ids", ",".join(map(str, p)))]) == 0
    shown = [json.loads(m) for m in re.findall(r"^output \d+: (\[.*\])$", capsys.readouterr().out, flags=re.M)]
    assert len(shown) == len(prompts)
    for prompt, got in zip(prompts, shown):
        tokens = list(prompt)
        for token in got:  # the written model's weights are small: equal logits are allowed for
            logits = plain.forward(raw, tensors, tokens)[-1]
            assert float(logits.max() - logits[token]) <= 1e-4 * float(logits.abs().max().clamp_min(1.0))
            tokens.append(token)
    assert cli.main(["engine", "kv-size", "--model", str(folder), "--dtype", "bfloat16", "--max-model-len", "64",
                     "--block-size", str(page)]) == 0
    sizing = capsys.readouterr().out
    sizing = json.loads(sizing[sizing.index("{"):])
    assert len(sizing["num_blocks"]) == 2 and sizing["activation_bytes"] > 0
