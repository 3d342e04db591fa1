"""Nagezen on the GPU against the plain implementation (tests/plain_nagezen.py, float64): every mechanism's kernels
alone -- with inputs made so that one key, one edge of a window or one kept token decides the result --, then whole
models: prompts whole, decoded token by token, in portions down to two tokens, unequal requests in one batch, pages and
state slots that are used again, long decoding, greedy generation through the entry point and the scheduler -- in 32-bit
and in bfloat16, on configurations that differ in every size (tests/nagezen_models.py)."""
import itertools
import math
import types

import numpy as np
import pytest
import torch

import helpers
import nagezen_models
import plain_nagezen as plain

pytestmark = pytest.mark.gpu

# A row of logits may differ from the plain row by this fraction of the plain row's root mean square (the errors' root
# mean square over the vocabulary), and no single logit by more than ten times that.
ROW_RMS = {"float32": 2e-5, "bfloat16": 6e-2}
LENGTHS = {"A": [1, 2, 9, 70, 150], "B": [3, 33, 64, 129], "C": [1, 17, 140], "D": [1, 3, 90, 200], "E": [2, 70, 131]}


def close_rows(got, where, plain_logits, dtype, label, factor=1.0):
    assert set(got) == set(where), f"{label}: rows produced {len(got)}, rows expected {len(where)}"
    limit, worst = ROW_RMS[dtype] * factor, 0.0
    for key in sorted(where):
        rid, pos = where[key]
        ref, row = plain_logits[rid][pos], got[key]
        assert np.all(np.isfinite(row)), f"{label}: non-finite logits at step {key[0]}, request {rid}, position {pos}"
        err, size = row - ref, float(np.sqrt(np.mean(ref * ref)))
        rms = float(np.sqrt(np.mean(err * err))) / size
        assert rms <= limit and float(np.abs(err).max()) <= 10 * limit * size, (
            f"{label}: first wrong row at step {key[0]}, request {rid}, position {pos}: errors' rms {rms:.3g} of the "
            f"row's (limit {limit:.3g}), largest {np.abs(err).max():.3g} of {size:.3g}")
        worst = max(worst, rms)
    return worst


@pytest.fixture(scope="module")
def setups(tmp_path_factory):
    """(name, dtype) -> (folder, requests, plain logits of every request)."""
    tmp, made = tmp_path_factory.mktemp("nagezen"), {}

    def get(name, dtype):
        key = (name, dtype)
        if key not in made:
            draw = dict(query_factor=1.2) if dtype == "bfloat16" else {}
            folder = nagezen_models.write_folder(tmp, name, dtype, drop_rank=name in ("B", "C"), **draw)
            model = plain.PlainNagezen(folder)
            requests = {f"r{i}": helpers.random_ids(n, model.cfg["vocab"], 400 + i) for i, n in enumerate(LENGTHS[name])}
            logits = {rid: model.forward(ids).numpy() for rid, ids in requests.items()}
            made[key] = (folder, requests, logits)
        return made[key]
    return get


def executor(folder, dtype, num_pages, page_tokens, max_requests=4, max_tokens=0, **kw):
    from bare_cuda_4gib_amd.engine import Executor, load_model
    model, _ = load_model(folder, dtype, "cuda:0")
    ex = Executor(model, num_pages=num_pages, max_requests=max_requests, max_tokens=max_tokens or num_pages * page_tokens,
                  page_tokens=page_tokens, poison=True, **kw)
    ex.cache.shuffle_free_pages(5)
    return ex


CASES = [(n, d) for n in sorted(nagezen_models.CONFIGS) for d in ("float32", "bfloat16")]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompts(setups, name, dtype):
    folder, requests, logits = setups(name, dtype)
    steps, where = helpers.trace_whole(requests)
    got = helpers.replay_in_process(executor(folder, dtype, 20, 16), steps)
    close_rows(got, where, logits, dtype, f"whole {name} {dtype}")


@pytest.mark.parametrize("name,dtype", CASES)
def test_prefill_against_decoding_token_by_token(setups, name, dtype):
    """Most of a request in one step, its last 40 tokens one by one (captured decode steps: a state must move once a
    step, also in the step that is captured; the windows pass over decoded tokens)."""
    folder, requests, logits = setups(name, dtype)
    steps, where = helpers.trace_tail_one_by_one(requests, tail=40)
    got = helpers.replay_in_process(executor(folder, dtype, 20, 16), steps)
    close_rows(got, where, logits, dtype, f"tail {name} {dtype}")


@pytest.mark.parametrize("name,dtype", CASES)
def test_portions_down_to_two_tokens(setups, name, dtype):
    folder, requests, logits = setups(name, dtype)
    for seed, sizes in ((1, (17, 2, 5, 64, 3, 2, 31, 9)), (2, (2, 2, 3, 16, 15, 1, 33, 70))):
        steps, where = helpers.trace_portions(requests, seed, sizes)
        got = helpers.replay_in_process(executor(folder, dtype, 20, 16), steps)
        close_rows(got, where, logits, dtype, f"portions {name} {dtype} {seed}")


@pytest.mark.parametrize("name,dtype", CASES)
def test_mixed_batches_with_pages_and_slots_used_again(setups, name, dtype):
    """Up to three live requests in three state slots and a pool just large enough: portions beside decoded tokens,
    requests left out of steps, pages and slots handed to the next request without being cleared by anyone but the
    admission (unowned pages hold NaN)."""
    folder, requests, logits = setups(name, dtype)
    many = dict(requests)
    many.update({rid + "again": ids for rid, ids in requests.items()})            # the same requests once more, in other slots
    plain_logits = dict(logits)
    plain_logits.update({rid + "again": logits[rid] for rid in requests})
    for seed in (3, 4):
        steps, where, peak = helpers.trace_mixed(many, seed, max_live=3, tail=10, page_tokens=16)
        ex = executor(folder, dtype, peak // 16, 16, max_requests=3, max_tokens=208)
        got = helpers.replay_in_process(ex, steps)
        close_rows(got, where, plain_logits, dtype, f"mixed {name} {dtype} {seed}")
        assert ex.cache.pages_in_use() == 0 and ex.cache.free_slots == 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_in_one_batch_against_each_alone(setups, dtype):
    from bare_cuda_4gib_amd.engine import StepEntry
    folder, requests, _ = setups("A", dtype)
    ex = executor(folder, dtype, 40, 16, max_requests=5)
    alone = {}
    for rid, ids in requests.items():
        ex.admit(rid)
        alone[rid] = ex.step([StepEntry(rid, ids, list(range(len(ids))))]).cpu().numpy()
        ex.release(rid)
    for rid in requests:
        ex.admit(rid)
    together = ex.step([StepEntry(rid, ids, list(range(len(ids)))) for rid, ids in requests.items()]).cpu().numpy()
    at = 0
    for rid, ids in requests.items():
        rows = together[at:at + len(ids)]
        at += len(ids)
        size = float(np.sqrt(np.mean(alone[rid] ** 2)))
        assert float(np.abs(rows - alone[rid]).max()) <= (1e-5 if dtype == "float32" else 5e-2) * size, rid


@pytest.mark.parametrize("name", ["A", "C"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_the_first_tokens(setups, name, dtype):
    """Two tokens, then 300 one by one over pages of 16: the states, the rotations and the windows far from the start,
    the kept first tokens long after the window has left them."""
    from bare_cuda_4gib_amd.engine import StepEntry
    folder, _, _ = setups(name, dtype)
    model = plain.PlainNagezen(folder)
    ids = helpers.random_ids(302, model.cfg["vocab"], 9)
    want = model.forward(ids).numpy()
    ex = executor(folder, dtype, 19, 16, max_requests=2)
    ex.admit("r")
    got = {}
    rows = ex.step([StepEntry("r", ids[:2], [0, 1])]).cpu().numpy()
    got[(0, 0)], got[(0, 1)] = rows[0], rows[1]
    for p in range(2, len(ids)):
        got[(0, p)] = ex.step([StepEntry("r", [ids[p]], [0])]).cpu().numpy()[0]
    where = {(0, p): ("r", p) for p in range(len(ids))}
    close_rows(got, where, {"r": want}, dtype, f"long decoding {name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_between_the_kept_tokens_and_the_window_go_back(setups, dtype):
    """A request four times as long as its pool: the pages that hold the kept first tokens stay, those the window has
    passed go back and are written again, and every row still equals the plain one."""
    from bare_cuda_4gib_amd.engine import StepEntry
    folder, _, _ = setups("E", dtype)
    model = plain.PlainNagezen(folder)
    ids = helpers.random_ids(260, model.cfg["vocab"], 19)
    want = model.forward(ids).numpy()
    ex = executor(folder, dtype, 10, 8, max_requests=2, max_tokens=320)      # 80 tokens of pages for 260 tokens
    ex.admit("r")
    got, where, at, n = {}, {}, 0, 0
    for size in itertools.cycle([5, 1, 1, 8, 3, 1, 16, 2]):
        size = min(size, len(ids) - at)
        rows = ex.step([StepEntry("r", ids[at:at + size], list(range(size)))]).cpu().numpy()
        for i in range(size):
            got[(n, i)], where[(n, i)] = rows[i], ("r", at + i)
        at, n = at + size, n + 1
        assert ex.cache.pages_in_use() <= 20          # (two groups of ten pages)
        if at == len(ids):
            break
    close_rows(got, where, {"r": want}, dtype, f"pool smaller than the request {dtype}")
    ex.release("r")
    assert ex.cache.pages_in_use() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point_and_the_scheduler(setups, dtype):
    from bare_cuda_4gib_amd.engine import Engine, generate_batch
    folder, _, _ = setups("A", dtype)
    model = plain.PlainNagezen(folder)
    prompts = [helpers.random_ids(n, model.cfg["vocab"], 50 + n) for n in (1, 5, 21, 40)]
    engine = Engine(folder, max_tokens=96, max_seqs=3, dtype=dtype, page_tokens=16, prefill_chunk=16)   # four requests, three slots
    together = generate_batch(engine, prompts, 24)
    margin = 1e-4 if dtype == "float32" else 0.3
    for prompt, tokens in zip(prompts, together):
        assert len(tokens) == 24
        full = model.forward(list(prompt) + list(tokens)).numpy()
        for i, tok in enumerate(tokens):                # every chosen token is the plain best, or within a near-tie of it
            row = full[len(prompt) - 1 + i]
            assert float(row.max() - row[tok]) <= margin, f"token {i} ({tok}) lies {row.max() - row[tok]:.4g} below the plain best"
    stats = engine.stats()
    assert stats["kv_pages_used"] == 0 and stats["running"] == 0


def test_the_command_line_generates_from_a_folder(setups):
    """bin/llm-infer over a Nagezen folder: the architecture is chosen by config.json, ids in, ids out."""
    import os
    import subprocess
    import sys
    folder, _, _ = setups("B", "float32")
    model = plain.PlainNagezen(folder)
    prompt = helpers.random_ids(9, model.cfg["vocab"], 4)
    proc = subprocess.run([sys.executable, os.path.join(helpers.ROOT, "bin", "llm-infer"), "--model", folder, "--prompt",
                           ",".join(map(str, prompt)), "--tokens", "6", "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    tokens = [int(t) for t in proc.stdout.strip().splitlines()[-1].split(":", 1)[1].split()]
    assert len(tokens) == 6
    full = model.forward(prompt + tokens).numpy()
    for i, tok in enumerate(tokens):
        row = full[len(prompt) - 1 + i]
        assert float(row.max() - row[tok]) <= 1e-4, (i, tok)


def test_the_replay_program_on_a_mixed_trace(setups, tmp_path):
    folder, requests, logits = setups("A", "float32")
    steps, where, peak = helpers.trace_mixed(requests, 8, max_live=4, tail=6, page_tokens=64)
    got = helpers.replay_subprocess(folder, "float32", steps, str(tmp_path / "out"), peak, nagezen_models.CONFIGS["A"]["vocab"])
    close_rows(got, where, logits, "float32", "bin/trace_run")


# ---- the kernels of each mechanism alone ---------------------------------------------------------------------------

DEV = "cuda:0"


def step_context(lengths, cached, slots):
    """What the kernels read of a step's context: request s brings lengths[s] rows after cached[s] tokens, in slot slots[s]."""
    starts = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    row_seq = np.concatenate([np.full(n, s, dtype=np.int32) for s, n in enumerate(lengths)])
    positions = np.concatenate([np.arange(c, c + n, dtype=np.int32) for c, n in zip(cached, lengths)])
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=DEV)      # noqa: E731
    return types.SimpleNamespace(
        n_tokens=int(starts[-1]), n_seqs=len(lengths), row_seq=i32(row_seq), positions=i32(positions), seq_start=list(starts),
        seq_ctx=list(cached), seq_slots=list(slots), seq_start_dev=i32(starts), seq_slots_dev=i32(slots), seq_ctx_dev=i32(cached),
        max_kv_len=int(max(c + n for c, n in zip(cached, lengths))), captured=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [1, 2, 5, 8, 11, 16])
@pytest.mark.parametrize("H", [37, 40])
def test_streams_are_read_written_and_filled(dtype, n, H):
    """The copies of the stream: the read with and without the norm, at chosen rows; the write from the OLD copies
    (a matrix far from symmetric, so that [from, to] the wrong way round shows), with the next read riding along."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(n)
    T = 7
    x0 = torch.randn(T, H)
    x = ops.streams_fill(x0.to(DEV), n)
    assert torch.equal(x.cpu(), x0[:, None, :].expand(T, n, H))
    x = torch.randn(T, n, H)
    read, write, mix = torch.randn(n), torch.randn(n), torch.randn(n, n)
    alpha, g, b = torch.tensor([0.6]), torch.randn(H), torch.randn(H) * 0.2
    u = torch.einsum("s,tsd->td", read.double(), x.double())
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    got = ops.streams_read(x.to(DEV), read.to(DEV), None, torch.float32).cpu().double()
    assert torch.allclose(got, u, atol=1e-5, rtol=1e-5)
    got = ops.streams_read(x.to(DEV), read.to(DEV), (alpha.to(DEV), g.to(DEV), b.to(DEV), 1.0), dtype).cpu().double()
    assert torch.allclose(got, plain.dynamic_tanh(u, alpha.double(), g.double(), b.double()), atol=tol, rtol=tol)
    rows = torch.tensor([4, 0, 4], dtype=torch.int32)
    got = ops.streams_read(x.to(DEV), None, (alpha.to(DEV), g.to(DEV), b.to(DEV), 3.0), torch.float32, rows=rows.to(DEV)).cpu().double()
    assert torch.allclose(got, 3.0 * plain.dynamic_tanh(x.double().sum(1)[rows.long()], alpha.double(), g.double(), b.double()), atol=1e-5, rtol=1e-5)
    y = torch.randn(T, H)
    want = torch.einsum("st,snd->tnd", mix.double(), x.double().transpose(0, 1)).transpose(0, 1) + write.double()[None, :, None] * y.double()[:, None, :]
    xd = x.to(DEV)
    assert ops.streams_write(xd, y.to(DEV), mix.to(DEV), write.to(DEV)) is None
    assert torch.allclose(xd.cpu().double(), want, atol=1e-5, rtol=1e-5)
    xd = x.to(DEV)
    nxt = ops.streams_write(xd, y.to(DEV), mix.to(DEV), write.to(DEV), read.to(DEV), (alpha.to(DEV), g.to(DEV), b.to(DEV), 1.0), dtype)
    assert torch.allclose(xd.cpu().double(), want, atol=1e-5, rtol=1e-5)
    u2 = torch.einsum("s,tsd->td", read.double(), want)
    assert torch.allclose(nxt.cpu().double(), plain.dynamic_tanh(u2, alpha.double(), g.double(), b.double()), atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("inter", [53, 56])
def test_clamped_gated_unit(dtype, inter):
    """Values on both sides of the limit in both branches: the gate is clamped from above only, the other branch on both
    sides, and one is added to it after the clamp."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(3)
    gu = (torch.randn(9, 2 * inter) * 3).to(dtype)
    for limit in (0.5, 2.5):
        got = ops.clamped_glu(gu.to(DEV), limit, 1.702).cpu().double()
        want = plain.clamped_glu(gu[:, :inter].double(), gu[:, inter:].double(), limit)
        tol = 1e-5 if dtype == torch.float32 else 1e-2
        assert torch.allclose(got, want, atol=tol, rtol=tol)
    assert float(plain.clamped_glu(torch.tensor([-9.0]), torch.tensor([0.0]), 2.5)) < -1e-6      # (no clamp below on the gate)


@pytest.mark.parametrize("scaling", [None, dict(factor=8.0, original=64, fast=16.0, slow=2.0), dict(factor=3.0, original=4096, fast=24.0, slow=1.5)])
@pytest.mark.parametrize("dims,base", [(2, 10.0), (8, 500.0), (40, 30000.0)])
def test_rotation_tables_far_from_the_start(scaling, dims, base):
    from bare_cuda_4gib_amd.engine.spec import PartSpec
    from bare_cuda_4gib_amd.parts import build_part
    positions = torch.tensor([0, 1, 2, 63, 64, 1000, 70001, 1 << 20], dtype=torch.int32)
    part = build_part("position", PartSpec("rotary", dict(theta=base, dim=dims, scaling=scaling)))
    ctx = types.SimpleNamespace(positions=positions.to(DEV), shared=lambda key, make: make())
    table = part.table(ctx).cpu().double()
    cos, sin = plain.half_rotation_angles(positions, dims, base, scaling)
    assert torch.allclose(table[..., 0], cos, atol=2e-7, rtol=0) and torch.allclose(table[..., 1], sin, atol=2e-7, rtol=0)
    if scaling is not None and dims >= 8:
        plain_cos, _ = plain.half_rotation_angles(positions, dims, base, None)
        assert float((cos - plain_cos).abs().max()) > 0.1                                         # (the scaling is not a no-op here)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,half", [(3, 8, 2), (2, 48, 24), (5, 7, 0), (1, 130, 40), (4, 10, 5)])
def test_heads_are_biased_normed_rotated_scaled_and_written_to_their_slots(dtype, heads, dim, half):
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(dim)
    T, P = 6, 4
    wide = torch.randn(T, heads * dim + 11).to(dtype)                  # the heads are a part of wider rows
    x = wide[:, 5:5 + heads * dim]
    bias, w = torch.randn(heads * dim), torch.randn(dim) + 1.0
    positions = torch.tensor([0, 1, 2, 1000, 70001, 3], dtype=torch.int32)
    table = None
    cos = sin = torch.zeros(T, 0, dtype=torch.float64)
    if half:
        cos, sin = plain.half_rotation_angles(positions, 2 * half, 77.0, None)
        table = torch.stack([cos, sin], dim=-1).float().to(DEV)
    v = (x.double() + bias.double()).view(T, heads, dim)
    want = plain.half_rotation(plain.unit_rms(v, 1e-4) * w.double(), cos, sin) * 0.37
    out = torch.zeros(T, heads, dim, device=DEV)
    ops.heads_prepare(wide.to(DEV)[:, 5:5 + heads * dim], heads, dim, out, bias=bias.to(DEV), norm_weight=w.to(DEV), eps=1e-4, table=table, factor=0.37)
    assert torch.allclose(out.cpu().double(), want, atol=2e-5, rtol=2e-5)
    # no norm, no bias; into the pages of a cache through a slot map
    slot_map = torch.tensor([9, 2, 0, 7, 5, 11], dtype=torch.int32)
    cache = torch.zeros(3, heads, P, dim, dtype=dtype, device=DEV)
    ops.heads_prepare(wide.to(DEV)[:, 5:5 + heads * dim], heads, dim, cache, table=table, slot_map=slot_map.to(DEV), page_tokens=P)
    want = plain.half_rotation(x.double().view(T, heads, dim), cos, sin)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    flat = cache.cpu().double().permute(0, 2, 1, 3).reshape(3 * P, heads, dim)
    for t in range(T):
        assert torch.allclose(flat[slot_map[t]], want[t], atol=tol, rtol=tol), t
    assert float(flat[[1, 3, 4, 6, 8, 10]].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,vdim", [(3, 12), (2, 70), (1, 200)])
def test_heads_are_normed_and_gated(dtype, heads, vdim):
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(vdim)
    T = 5
    o, w = torch.randn(T, heads, vdim) * 4, torch.randn(vdim) + 1
    wide = torch.randn(T, heads * vdim + 6).to(dtype)
    gate = wide[:, 6:]
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    got = ops.heads_finish(o.to(DEV), dtype, weight=w.to(DEV), eps=1e-3, gate=wide.to(DEV)[:, 6:], act=ops.ACT_SILU).cpu().double()
    want = (plain.unit_rms(o.double(), 1e-3) * w.double()).reshape(T, -1) * plain.silu(gate.double())
    assert torch.allclose(got, want, atol=tol, rtol=tol)
    got = ops.heads_finish(o.to(DEV), torch.float32, eps=1e-3, factor=0.4).cpu().double()
    assert torch.allclose(got, plain.unit_rms(o.double(), 1e-3).reshape(T, -1) * 0.4, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,vdim", [(3, 5, 12), (2, 40, 70), (1, 72, 7), (1, 130, 33), (2, 64, 128), (2, 24, 20)])
@pytest.mark.parametrize("per_channel", [False, True])
def test_decayed_state_over_portions(dtype, heads, dim, vdim, per_channel):
    """Two requests of unequal length in portions of 1 to 200 rows (one chunk, several chunks, chunks' edges), in state
    slots that held something else before; decays from 0 to 1; the state after the last portion is the plain one."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(dim + vdim)
    lengths = [330, 77]
    seqs = []
    for T in lengths:
        q, k, v = torch.randn(T, heads * dim).to(dtype), (torch.randn(T, heads * dim) / math.sqrt(dim)).to(dtype), torch.randn(T, heads * vdim).to(dtype)
        z = torch.randn(T, heads * dim) * 3 + 2
        seqs.append((q, k, v, z))
    z_bias, head_decay, tau = torch.randn(heads * dim), torch.tensor([1.0, 0.0, 0.96][:heads]), 3.0
    want, last = [], []
    for q, k, v, z in seqs:
        T = q.shape[0]
        if per_channel:
            decay = (torch.sigmoid(z.double() + z_bias.double()) ** (1.0 / tau)).view(T, heads, dim)
        else:
            decay = head_decay.double()[None, :, None].expand(T, heads, dim)
        outs = [plain.decayed_outer_products(q.double().view(T, heads, dim)[:, a] * 0.7, k.double().view(T, heads, dim)[:, a],
                                             v.double().view(T, heads, vdim)[:, a], decay[:, a]) for a in range(heads)]
        want.append(torch.stack(outs, dim=1))
    state = torch.full((4, heads, dim, vdim), 9.0, device=DEV)
    slots = [2, 0]
    for s in slots:
        state[s].zero_()                                  # what admission does
    done, got = [0, 0], [[], []]
    sizes = itertools.cycle([3, 1, 64, 65, 1, 128, 2, 200, 1, 7])
    while any(d < n for d, n in zip(done, lengths)):
        live = [s for s in (0, 1) if done[s] < lengths[s]]
        lens = [min(next(sizes), lengths[s] - done[s]) for s in live]
        ctx = step_context(lens, [done[s] for s in live], [slots[s] for s in live])
        batch = types.SimpleNamespace(n_seqs=len(lens), seq_start=ctx.seq_start)
        base, total = ops.decay_scan_chunks(batch)
        cut = lambda i: torch.cat([seqs[s][i][done[s]:done[s] + n] for s, n in zip(live, lens)]).to(DEV)      # noqa: E731
        kw = dict(z=cut(3), z_bias=z_bias.to(DEV), inv_tau=1.0 / tau) if per_channel else dict(head_decay=head_decay.to(DEV))
        out = ops.decay_scan(cut(0), cut(1), cut(2), state, ctx, heads, dim, vdim, q_scale=0.7,
                             chunk_base=torch.tensor(base, dtype=torch.int32, device=DEV), n_chunks=total, **kw).cpu()
        at = 0
        for s, n in zip(live, lens):
            got[s].append(out[at:at + n])
            at, done[s] = at + n, done[s] + n
    for s in (0, 1):
        size = float(want[s].abs().max())
        assert torch.allclose(torch.cat(got[s]).double(), want[s], atol=2e-5 * size, rtol=2e-5), (s, per_channel)
    assert float(state[1].min()) == 9.0 and float(state[3].max()) == 9.0          # other requests' slots are left alone


def paged(rows_k, rows_v, pages, P, dtype, n_pages):
    """Caches [n_pages + 1, heads, P, size] filled with NaN but for the given rows ([n, heads, size]) in the given pages."""
    k = torch.full((n_pages + 1, rows_k.shape[1], P, rows_k.shape[2]), float("nan"), dtype=dtype, device=DEV)
    v = torch.full((n_pages + 1, rows_v.shape[1], P, rows_v.shape[2]), float("nan"), dtype=dtype, device=DEV)
    for j in range(rows_k.shape[0]):
        k[pages[j // P], :, j % P] = rows_k[j].to(dtype).to(DEV)
        v[pages[j // P], :, j % P] = rows_v[j].to(dtype).to(DEV)
    return k, v


def plain_maps(q, keys, values, pos, G, maps, scale, window, keep_first, lam):
    """The plain result for one row at position ``pos``: q [H, maps, d], keys [n, G * maps, d], values [n, G, e]."""
    H = q.shape[0]
    seen = [j for j in range(pos + 1) if plain.visible(pos, j, window, keep_first)]
    out, weights = [], []
    for a in range(H):
        g = a // (H // G)
        per_map = []
        for m in range(maps):
            s = (keys[seen, g * maps + m].double() @ q[a, m].double()) * scale
            w = torch.softmax(s, 0)
            per_map.append(w)
        o = per_map[0] @ values[seen, g].double()
        if maps == 2:
            o = o - lam * (per_map[1] @ values[seen, g].double())
        out.append(o)
        weights.append(per_map)
    return torch.stack(out), weights, seen


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(4, 2, 2, 12, 20), (3, 3, 1, 10, 70), (6, 1, 2, 44, 100), (2, 1, 2, 7, 130), (2, 2, 2, 72, 200), (4, 1, 1, 128, 64)])
@pytest.mark.parametrize("needle", [0, 7, 8, 63, 64, 120, 199])
def test_attention_finds_one_key_among_hundreds(dtype, needle, sizes):
    """200 cached keys in scattered pages of 8, no window; one key, far back, at a page's border or the row's own, is
    made to score far above the others in the first map of one head: that map's weight goes there, the result equals the
    plain one for every head.  As a decoded token and as the last rows of a prompt portion."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(needle)
    (H, G, maps, d, e), n, P, scale, lam = sizes, 200, 8, 0.3, 0.35
    keys, values = (torch.randn(n, G * maps, d) * 0.3).to(dtype).float(), torch.randn(n, G, e).to(dtype).float()
    q = torch.randn(H, maps, d)
    mark = min(1, H - 1)
    keys[needle, (mark // (H // G)) * maps] = (q[mark, 0] / float(q[mark, 0] @ q[mark, 0]) * 14.0 / scale).to(dtype).float()
    pages = torch.randperm(40)[:n // P]
    k_cache, v_cache = paged(keys, values, pages, P, dtype, 40)
    table = pages.to(torch.int32).view(1, -1).to(DEV)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for lengths, cached in (([1], [n - 1]), ([6], [n - 6])):
        ctx = step_context(lengths, cached, [0])
        qs = q.view(1, H, maps, d).repeat(lengths[0], 1, 1, 1).contiguous().to(DEV)
        got = ops.attention_maps(qs, k_cache, v_cache, table, ctx, torch.float32, H, G, maps, d, e, 0, 0, scale, lam=lam).cpu().double()
        for r in range(lengths[0]):
            pos = cached[0] + r
            want, weights, seen = plain_maps(q, keys, values, pos, G, maps, scale, 0, 0, lam)
            assert torch.allclose(got[r].view(H, e), want, atol=tol * float(want.abs().max()), rtol=tol), (needle, pos)
            if needle <= pos:
                assert float(weights[mark][0][seen.index(needle)]) > 0.9


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,keep_first", [(50, 0), (50, 5), (9, 3), (6, 10), (64, 64), (65, 1)])
@pytest.mark.parametrize("where", ["window_in", "window_out", "first_in", "first_out"])
def test_attention_at_the_edges_of_the_window_and_of_the_kept_tokens(dtype, window, keep_first, where):
    """A key made to stand out just inside the window takes the weight; the same key one place further back is not seen
    at all; the last kept first token takes it however far the window has moved, the token after it does not -- as a
    decoded token and in a portion whose rows' windows begin at different keys, over pages of 16."""
    from bare_cuda_4gib_amd.csrc import ops
    if where.startswith("first") and keep_first == 0:
        pytest.skip("no kept tokens in this case")
    torch.manual_seed(window)
    H, G, maps, d, e, n, P, scale, lam = 4, 2, 2, 12, 20, 150, 16, 0.3, 0.4
    keys, values = (torch.randn(n, G * maps, d) * 0.3).to(dtype).float(), torch.randn(n, G, e).to(dtype).float()
    q = torch.randn(H, maps, d)
    pos_last = n - 1
    needle = {"window_in": pos_last - window + 1, "window_out": pos_last - window, "first_in": keep_first - 1, "first_out": keep_first}[where]
    for m in range(maps):        # both maps of the first key/value head point at the needle (head 0 reads it)
        keys[needle, m] = (q[0, m] / float(q[0, m] @ q[0, m]) * 14.0 / scale).to(dtype).float()
    pages = torch.randperm(20)[:-(-n // P)]
    k_cache, v_cache = paged(keys, values, pages, P, dtype, 20)
    table = pages.to(torch.int32).view(1, -1).to(DEV)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for lengths, cached in (([1], [n - 1]), ([5], [n - 5])):
        ctx = step_context(lengths, cached, [0])
        qs = q.view(1, H, maps, d).repeat(lengths[0], 1, 1, 1).contiguous().to(DEV)
        got = ops.attention_maps(qs, k_cache, v_cache, table, ctx, torch.float32, H, G, maps, d, e, window, keep_first, scale,
                                 lam=lam, normalize=True, eps=1e-5, factor=0.6).cpu().double()
        for r in range(lengths[0]):
            pos = cached[0] + r
            want, weights, seen = plain_maps(q, keys, values, pos, G, maps, scale, window, keep_first, lam)
            want = plain.unit_rms(want, 1e-5) * 0.6
            assert torch.allclose(got[r].view(H, e), want, atol=tol * float(want.abs().max()), rtol=tol), (where, pos)
            if pos == pos_last:
                inside = where.endswith("_in") or (where == "first_out" and pos - needle < window) or (where == "window_out" and needle < keep_first)
                assert (needle in seen) == inside
                if inside:
                    assert float(weights[0][0][seen.index(needle)]) > 0.9


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_of_the_first_tokens_and_of_unequal_requests(dtype):
    """Three requests in one step -- the first token of a sequence, a portion from position 0, a decoded token far in --
    each with a block table of its own, with gates: every row equals the plain one."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(8)
    H, G, maps, d, e, P, scale, lam, window, keep = 3, 3, 2, 10, 6, 4, 0.5, 0.2, 5, 2
    lengths, cached = [1, 9, 1], [0, 0, 30]
    n_pages = 24
    k_cache = torch.full((n_pages + 1, G * maps, P, d), float("nan"), dtype=dtype, device=DEV)
    v_cache = torch.full((n_pages + 1, G, P, e), float("nan"), dtype=dtype, device=DEV)
    perm = torch.randperm(n_pages)
    tables, seqs, at = torch.full((3, 8), -1, dtype=torch.int32), [], 0
    for s, (new, old) in enumerate(zip(lengths, cached)):
        n = new + old
        keys, values = (torch.randn(n, G * maps, d)).to(dtype).float(), torch.randn(n, G, e).to(dtype).float()
        pages = perm[at:at + -(-n // P)]
        at += len(pages)
        tables[s, :len(pages)] = pages.to(torch.int32)
        for j in range(n):
            k_cache[pages[j // P], :, j % P] = keys[j].to(dtype).to(DEV)
            v_cache[pages[j // P], :, j % P] = values[j].to(dtype).to(DEV)
        seqs.append((keys, values))
    ctx = step_context(lengths, cached, [0, 1, 2])
    q = torch.randn(sum(lengths), H, maps, d)
    gate = torch.randn(sum(lengths), H * e).to(dtype)
    got = ops.attention_maps(q.to(DEV), k_cache, v_cache, tables.to(DEV), ctx, torch.float32, H, G, maps, d, e, window, keep, scale,
                             lam=lam, normalize=True, eps=1e-6, factor=0.9, gate=gate.to(DEV), act=ops.ACT_SIGMOID).cpu().double()
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    row = 0
    for s, (new, old) in enumerate(zip(lengths, cached)):
        for i in range(new):
            want, _, _ = plain_maps(q[row], seqs[s][0], seqs[s][1], old + i, G, maps, scale, window, keep, lam)
            want = (plain.unit_rms(want, 1e-6) * 0.9).reshape(-1) * torch.sigmoid(gate[row].double())
            assert torch.allclose(got[row], want, atol=tol, rtol=tol), (s, i)
            row += 1
