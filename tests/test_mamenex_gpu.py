"""Mamenex on the GPU against the plain implementation (tests/plain_mamenex.py, float64): every mechanism's kernels
alone, then whole models -- prompts whole, decoded token by token, in portions down to two tokens, unequal requests
in one batch, pages and state slots that are used again, long decoding, greedy generation through the entry point and
the scheduler -- in 32-bit and in bfloat16, on configurations that differ in every size (tests/mamenex_models.py)."""
import itertools
import math
import types

import numpy as np
import pytest
import torch

import helpers
import mamenex_models
import plain_mamenex as plain

pytestmark = pytest.mark.gpu

# A row of logits may differ from the plain row by this fraction of the plain row's root mean square (the errors'
# root mean square over the vocabulary), and no single logit by more than ten times that.  32-bit: float arithmetic
# against float64 through up to four layers with peaked attention.  bfloat16: activations between kernels carry 8 bits; peaked attention multiplies what the layers before have
# left (two keys that score alike change places), so the bfloat16 folders are drawn with smaller query weights.
ROW_RMS = {"float32": 2e-5, "bfloat16": 5e-2}
LENGTHS = {"P": [1, 2, 9, 70, 150], "Q": [3, 33, 64, 129], "R": [1, 17, 140], "S": [1, 5, 40, 131], "T": [1, 3, 90], "U": [2, 70], "V": [1, 4, 75]}


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
    """(name, dtype, variant) -> (folder, requests, plain logits of every request)."""
    tmp, made = tmp_path_factory.mktemp("mamenex"), {}

    def get(name, dtype, variant=""):
        key = (name, dtype, variant)
        if key not in made:
            draw = dict(sink_mean=4.0, query_factor=1.5) if variant == "sink" else {}
            if dtype == "bfloat16":
                draw["query_factor"] = 1.2
            folder = mamenex_models.write_folder(tmp, name, dtype, tag=variant, **draw)
            config, weights = plain.load_folder(folder)
            requests = {f"r{i}": helpers.random_ids(n, config["vocab"], 300 + i) for i, n in enumerate(LENGTHS[name])}
            logits = {rid: plain.forward(config, weights, ids).numpy() for rid, ids in requests.items()}
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


CASES = [(n, d) for n in sorted(mamenex_models.CONFIGS) for d in ("float32", "bfloat16")]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompts(setups, name, dtype):
    folder, requests, logits = setups(name, dtype)
    steps, where = helpers.trace_whole(requests)
    got = helpers.replay_in_process(executor(folder, dtype, 20, 16), steps)
    close_rows(got, where, logits, dtype, f"whole {name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_sink_that_takes_most_of_the_weight(setups, dtype):
    """Sinks drawn around 4: most of every row's weight goes to the sink, so leaving it out, scaling it or counting it
    per key would change every logit."""
    folder, requests, logits = setups("P", dtype, "sink")
    config, weights = plain.load_folder(folder)
    without = dict(weights)
    for n in (1, 2):
        without[f"l{n}.mix.sink"] = torch.full_like(weights[f"l{n}.mix.sink"], -1e4)
    ids = requests["r3"]
    assert float((plain.forward(config, without, ids) - torch.from_numpy(logits["r3"])).abs().max()) > 0.5
    steps, where = helpers.trace_tail_one_by_one(requests, tail=20)
    got = helpers.replay_in_process(executor(folder, dtype, 20, 16), steps)
    close_rows(got, where, logits, dtype, f"sink {dtype}")


@pytest.mark.parametrize("name,dtype", CASES)
def test_prefill_against_decoding_token_by_token(setups, name, dtype):
    """Most of a request in one step, its last 40 tokens one by one (captured decode steps: the state of the recurrence
    and the convolutions' tails must move once a step, also in the step that is captured)."""
    folder, requests, logits = setups(name, dtype)
    steps, where = helpers.trace_tail_one_by_one(requests, tail=40)
    got = helpers.replay_in_process(executor(folder, dtype, 20, 16), steps)
    close_rows(got, where, logits, dtype, f"tail {name} {dtype}")


@pytest.mark.parametrize("name,dtype", CASES)
def test_portions_down_to_two_tokens(setups, name, dtype):
    folder, requests, logits = setups(name, dtype)
    for seed, sizes in ((1, (17, 2, 5, 64, 3, 2, 31, 9)), (2, (2, 2, 3, 16, 15, 1, 33))):
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
        ex = executor(folder, dtype, peak // 16, 16, max_requests=3, max_tokens=160)
        got = helpers.replay_in_process(ex, steps)
        close_rows(got, where, plain_logits, dtype, f"mixed {name} {dtype} {seed}")
        assert ex.cache.pages_in_use() == 0 and ex.cache.free_slots == 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_in_one_batch_against_each_alone(setups, dtype):
    from bare_cuda_4gib_amd.engine import StepEntry
    folder, requests, _ = setups("Q", dtype)
    ex = executor(folder, dtype, 40, 16, max_requests=4)
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_the_first_tokens(setups, dtype):
    """Two tokens, then 300 one by one over pages of 16: the recurrence's state and the rotations far from the start."""
    from bare_cuda_4gib_amd.engine import StepEntry
    folder, _, _ = setups("P", dtype)
    config, weights = plain.load_folder(folder)
    ids = helpers.random_ids(302, config["vocab"], 9)
    want = plain.forward(config, weights, ids).numpy()
    ex = executor(folder, dtype, 19, 16, max_requests=2)
    ex.admit("r")
    got = {}
    rows = ex.step([StepEntry("r", ids[:2], [0, 1])]).cpu().numpy()
    got[(0, 0)], got[(0, 1)] = rows[0], rows[1]
    for p in range(2, len(ids)):
        got[(0, p)] = ex.step([StepEntry("r", [ids[p]], [0])]).cpu().numpy()[0]
    where = {(0, p): ("r", p) for p in range(len(ids))}
    close_rows(got, where, {"r": want}, dtype, f"long decoding {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point_and_the_scheduler(setups, dtype):
    from bare_cuda_4gib_amd.engine import Engine, generate_batch
    folder, _, _ = setups("Q", dtype)
    config, weights = plain.load_folder(folder)
    prompts = [helpers.random_ids(n, config["vocab"], 50 + n) for n in (1, 5, 21, 40)]
    engine = Engine(folder, max_tokens=96, max_seqs=3, dtype=dtype, page_tokens=16, prefill_chunk=16)   # four requests, three slots
    together = generate_batch(engine, prompts, 24)
    margin = 1e-4 if dtype == "float32" else 0.25
    for prompt, tokens in zip(prompts, together):
        assert len(tokens) == 24
        full = plain.forward(config, weights, list(prompt) + list(tokens)).numpy()
        for i, tok in enumerate(tokens):                # every chosen token is the plain best, or within a near-tie of it
            row = full[len(prompt) - 1 + i]
            assert float(row.max() - row[tok]) <= margin, f"token {i} ({tok}) lies {row.max() - row[tok]:.4g} below the plain best"
    stats = engine.stats()
    assert stats["kv_pages_used"] == 0 and stats["running"] == 0


def test_the_command_line_generates_from_a_folder(setups):
    """bin/llm-infer over a Mamenex folder: the architecture is chosen by config.json, ids in, ids out."""
    import os
    import subprocess
    import sys
    folder, _, _ = setups("S", "float32")
    config, weights = plain.load_folder(folder)
    prompt = helpers.random_ids(9, config["vocab"], 4)
    proc = subprocess.run([sys.executable, os.path.join(helpers.ROOT, "bin", "llm-infer"), "--model", folder, "--prompt",
                           ",".join(map(str, prompt)), "--tokens", "6", "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    tokens = [int(t) for t in proc.stdout.strip().splitlines()[-1].split(":", 1)[1].split()]
    assert len(tokens) == 6
    full = plain.forward(config, weights, prompt + tokens).numpy()
    for i, tok in enumerate(tokens):
        row = full[len(prompt) - 1 + i]
        assert float(row.max() - row[tok]) <= 1e-4, (i, tok)


def test_the_replay_program_on_a_mixed_trace(setups, tmp_path):
    folder, requests, logits = setups("P", "float32")
    steps, where, peak = helpers.trace_mixed(requests, 8, max_live=4, tail=6, page_tokens=64)
    got = helpers.replay_subprocess(folder, "float32", steps, str(tmp_path / "out"), peak, mamenex_models.CONFIGS["P"]["vocab"])
    close_rows(got, where, logits, "float32", "bin/trace_run")


# ---- the kernels of each mechanism alone ---------------------------------------------------------------------------

def step_context(lengths, cached, slots):
    """What the kernels read of a step's context: request s brings lengths[s] rows after cached[s] tokens, in slot slots[s]."""
    dev = "cuda:0"
    starts = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    row_seq = np.concatenate([np.full(n, s, dtype=np.int32) for s, n in enumerate(lengths)])
    positions = np.concatenate([np.arange(c, c + n, dtype=np.int32) for c, n in zip(cached, lengths)])
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=dev)      # noqa: E731
    return types.SimpleNamespace(
        n_tokens=int(starts[-1]), n_seqs=len(lengths), row_seq=i32(row_seq), positions=i32(positions), seq_start=list(starts),
        seq_ctx=list(cached), seq_slots=list(slots), seq_start_dev=i32(starts), seq_slots_dev=i32(slots), seq_ctx_dev=i32(cached),
        max_kv_len=int(max(c + n for c, n in zip(cached, lengths))), captured=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_convolution_over_portions(dtype, taps):
    """Two requests of unequal length fed in portions of 1 to 7 rows, in slots that held another request's tail before:
    every row equals the convolution of the whole sequence."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(taps)
    C, dev = 37, "cuda:0"
    w, b_in, b_out = torch.randn(C, taps), torch.randn(C), torch.randn(C)
    seqs = [torch.randn(23, C).to(dtype), torch.randn(11, C).to(dtype)]
    state = torch.full((4, taps - 1, C), 5.0, dtype=dtype, device=dev)
    slots = [2, 0]
    for s in slots:
        state[s].zero_()                                  # what admission does
    for add_input in (False, True):
        want = []
        for v in seqs:
            inputs = (v.double() + b_in.double()).to(dtype).double()          # the inputs as they are kept
            want.append(plain.causal_conv(inputs, w.double(), b_out.double()) + (v.double() if add_input else 0))
        done, got = [0, 0], [[], []]
        sizes = itertools.cycle([3, 1, 7, 2, 1, 1, 5, 4, 6, 2, 3, 7, 1, 2])
        st = state.clone()
        while any(d < len(v) for d, v in zip(done, seqs)):
            live = [s for s in (0, 1) if done[s] < len(seqs[s])]
            lens = [min(next(sizes), len(seqs[s]) - done[s]) for s in live]
            ctx = step_context(lens, [done[s] for s in live], [slots[s] for s in live])
            x = torch.cat([seqs[s][done[s]:done[s] + n] for s, n in zip(live, lens)]).to(dev)
            out = ops.causal_conv(x, w.t().contiguous().to(dev), st if taps > 1 else None, ctx, in_bias=b_in.to(dev), out_bias=b_out.to(dev),
                                  add_input=add_input).cpu()
            at = 0
            for s, n in zip(live, lens):
                got[s].append(out[at:at + n])
                at, done[s] = at + n, done[s] + n
        for s in (0, 1):
            tol = 1e-5 if dtype == torch.float32 else 3e-2
            assert torch.allclose(torch.cat(got[s]).double(), want[s], atol=tol, rtol=tol), (taps, add_input, s)
        if taps > 1:
            assert float(st[1].min()) == 5.0 and float(st[3].max()) == 5.0      # other requests' slots are left alone


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_added_to_the_stream_and_activation(dtype):
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(2)
    dev = "cuda:0"
    x, y, w = torch.randn(5, 77), (torch.randn(5, 77) * 3).to(dtype), torch.randn(77) * 0.3
    want = x.double() + plain.offset_rmsnorm(y.double(), w.double(), 1e-3)
    got = ops.rmsnorm_add(x.to(dev), y.to(dev), (1.0 + w).to(dev), 1e-3).cpu()
    assert torch.allclose(got.double(), want, atol=1e-5, rtol=1e-5)
    z, pq = (torch.randn(4000) * 3).to(dtype), torch.tensor([0.4, -0.8])
    got = ops.xielu(z.to(dev), pq.to(dev)).cpu().double()
    want = plain.xielu(z.double(), pq[0].double(), pq[1].double())
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert torch.allclose(got, want, atol=tol, rtol=tol)
    assert float(ops.xielu(torch.zeros(3, dtype=dtype, device=dev), pq.to(dev)).abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("blocks,width", [(1, 24), (3, 30), (2, 160)])
def test_recurrence_over_portions(dtype, blocks, width):
    """The gates, the decay and the state in float32, continued from portion to portion; a decay close to one
    (large lam) and close to zero both occur."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(width)
    dev, T, bs = "cuda:0", 350, width // blocks
    u, y = torch.randn(T, width).to(dtype), torch.randn(T, width).to(dtype)
    ra, ri = (torch.randn(blocks, bs, bs) / math.sqrt(bs)).to(dtype), (torch.randn(blocks, bs, bs) / math.sqrt(bs)).to(dtype)
    ra_b, ri_b, lam, y_b = torch.randn(width), torch.randn(width), torch.randn(width) * 3 - 2, torch.randn(width) * 0.3
    ud = u.double().view(T, blocks, bs)
    r = torch.sigmoid(torch.einsum("boi,tbi->tbo", ra.double(), ud).reshape(T, width) + ra_b.double())
    i = torch.sigmoid(torch.einsum("boi,tbi->tbo", ri.double(), ud).reshape(T, width) + ri_b.double())
    a = torch.exp(-8.0 * r * plain.softplus(lam.double()))
    S, want = torch.zeros(width, dtype=torch.float64), []
    for t in range(T):
        S = a[t] * S + torch.sqrt(1 - a[t] ** 2) * i[t] * u[t].double()
        want.append(S * plain.gelu_tanh(y[t].double() + y_b.double()))
    want = torch.stack(want)
    state = torch.full((3, width), 9.0, device=dev)
    state[1].zero_()
    got, at = [], 0
    for n in (1, 2, 40, 1, 1, 64, 3, 38, 200):
        ctx = step_context([n], [at], [1])
        got.append(ops.rglru(u[at:at + n].to(dev), y[at:at + n].to(dev), torch.cat([ra, ri], dim=1).contiguous().to(dev), ra_b.to(dev), ri_b.to(dev), lam.to(dev), y_b.to(dev), state, ctx).cpu())
        at += n
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(torch.cat(got).double(), want, atol=tol, rtol=tol)
    assert torch.allclose(state[1].cpu().double(), S, atol=1e-5, rtol=1e-5) and float(state[0].min()) == 9.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(3, 20, 12), (4, 48, 16), (20, 112, 16), (16, 512, 64), (8, 128, 64), (2, 256, 32), (33, 64, 64),
                                   (5, 32, 0), (1, 700, 100)])
@pytest.mark.parametrize("needle", [0, 7, 8, 31, 32, 120, 199])
def test_latent_attention_finds_one_key_among_hundreds(dtype, needle, sizes):
    """200 cached rows in scattered pages of 8; one row, far back, at a page's border or the row's own, is made to
    score far above the others for one head: that head's output is that row's latent, the others' are not, and all
    equal the plain softmax with a sink.  As a decoded token and as the last rows of a prompt portion; in sizes that
    the plain kernel serves and (bfloat16) in sizes of the matrix-core kernel, whose walks here are cut into parts."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(needle)
    (H, rank, rot), dev, n, P, scale = sizes, "cuda:0", 200, 8, 0.3
    rows = (torch.randn(n, rank + rot) * 0.3).to(dtype)
    q = torch.randn(H, rank + rot)
    mark = min(1, H - 1)
    rows[needle] = (q[mark] / float(q[mark] @ q[mark]) * 14.0 / scale).to(dtype)        # its score for that head: 14
    sink = torch.randn(H) + 1.0
    pages = torch.randperm(40)[:n // P]
    tensor_cores = dtype == torch.bfloat16 and ops.attention_latent_mfma_takes(torch.empty(8, dtype=dtype, device=dev), rank, rot)
    tol = 3e-2 if tensor_cores else 2e-5        # there the queries and the weights are rounded to bfloat16
    cache = torch.full((41, P, rank + rot), float("nan"), dtype=dtype, device=dev)
    for j in range(n):
        cache[pages[j // P], j % P] = rows[j].to(dev)
    table = pages.to(torch.int32).view(1, -1).to(dev)
    for lengths, cached in (([1], [n - 1]), ([6], [n - 6])):
        ctx = step_context(lengths, cached, [0])
        q_lat = q.view(1, H, -1).repeat(lengths[0], 1, 1).contiguous().to(dev)
        got = ops.attention_latent(q_lat, cache, sink.to(dev), table, ctx, H, rank, rot, P, 0, scale).cpu().double()
        for k in range(lengths[0]):
            pos = cached[0] + k
            for a in range(H):
                s = (rows[:pos + 1].double() @ q[a].double()) * scale
                w = plain.sink_softmax(s, float(sink[a]))
                want = w @ rows[:pos + 1, :rank].double()
                assert torch.allclose(got[k, a], want, atol=tol * float(want.abs().max()), rtol=tol), (needle, pos, a)
                if a == mark and needle <= pos:
                    assert float(w[needle]) > 0.9


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(3, 20, 12), (4, 48, 16), (16, 128, 32)])
@pytest.mark.parametrize("back", [49, 50])
def test_latent_attention_within_a_window(dtype, sizes, back):
    """The part takes a window as a parameter (this design sets none): with a window of 50 a row sees the 50 keys up to
    its own.  A key made to stand out 49 places back takes the weight, the same key 50 places back is not seen at all --
    as a decoded token and in a portion whose rows' windows begin at different keys."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(back)
    (H, rank, rot), dev, n, P, scale, window = sizes, "cuda:0", 130, 16, 0.3, 50
    rows = (torch.randn(n, rank + rot) * 0.3).to(dtype)
    q = torch.randn(H, rank + rot)
    needle = n - 1 - back
    rows[needle] = (q[0] / float(q[0] @ q[0]) * 14.0 / scale).to(dtype)
    pages = torch.randperm(20)[:-(-n // P)]
    cache = torch.full((21, P, rank + rot), float("nan"), dtype=dtype, device=dev)
    for j in range(n):
        cache[pages[j // P], j % P] = rows[j].to(dev)
    table = pages.to(torch.int32).view(1, -1).to(dev)
    tensor_cores = dtype == torch.bfloat16 and ops.attention_latent_mfma_takes(cache, rank, rot)
    tol = 3e-2 if tensor_cores else 2e-5
    for lengths, cached in (([1], [n - 1]), ([5], [n - 5])):
        ctx = step_context(lengths, cached, [0])
        q_lat = q.view(1, H, -1).repeat(lengths[0], 1, 1).contiguous().to(dev)
        got = ops.attention_latent(q_lat, cache, None, table, ctx, H, rank, rot, P, window, scale).cpu().double()
        for k in range(lengths[0]):
            pos = cached[0] + k
            lo = max(0, pos - window + 1)
            for a in range(H):
                s = (rows[lo:pos + 1].double() @ q[a].double()) * scale
                w = torch.softmax(s, 0)                       # (no sink here)
                want = w @ rows[lo:pos + 1, :rank].double()
                assert torch.allclose(got[k, a], want, atol=tol * float(want.abs().max()), rtol=tol), (back, pos, a)
                if a == 0 and lo <= needle:
                    assert float(w[needle - lo]) > 0.9


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_rows_are_normed_rotated_and_written_to_their_slots(dtype):
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(4)
    dev, T, H, dn, dr, rank, dims, base, P = "cuda:0", 5, 2, 6, 10, 9, 6, 77.0, 4
    q, dkv, g = torch.randn(T, H * (dn + dr)).to(dtype), torch.randn(T, rank + dr).to(dtype), torch.randn(rank)
    positions = torch.tensor([0, 1, 2, 1000, 70001], dtype=torch.int32)
    slot_map = torch.tensor([9, 2, 0, 7, 5], dtype=torch.int32)
    cache = torch.zeros(3, P, rank + dr, dtype=dtype, device=dev)
    q_lat = torch.zeros(T, H, rank + dr, device=dev)
    angles = ops.latent_angles(positions.to(dev), dims, base)
    ops.latent_prepare(q.to(dev), dkv.to(dev), g.to(dev), 1e-4, angles, slot_map.to(dev), cache, q_lat, H, dn, dr, rank, dims)
    c = plain.plain_rmsnorm(dkv[:, :rank].double(), g.double(), 1e-4)
    kr = plain.interleaved_rotation(dkv[:, rank:].double(), positions.long(), base, dims)
    qr = plain.interleaved_rotation(q.double().view(T, H, dn + dr)[..., dn:], positions.long(), base, dims)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    flat = cache.view(-1, rank + dr).cpu().double()
    for t in range(T):
        assert torch.allclose(flat[slot_map[t]], torch.cat([c[t], kr[t]]), atol=tol, rtol=tol), t
    assert torch.allclose(q_lat[..., rank:].cpu().double(), qr, atol=1e-5, rtol=1e-5)       # float32 whatever the storage
    assert float(q_lat[..., :rank].abs().max()) == 0.0 and float(flat[[1, 3, 4, 6, 8, 10, 11]].abs().max()) == 0.0


@pytest.mark.parametrize("dtypes", [(torch.float32, torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16, torch.float32),
                                    (torch.float32, torch.bfloat16, torch.bfloat16)])
def test_a_product_per_head(dtypes):
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(6)
    dev, T, H, k, n = "cuda:0", 70, 3, 21, 67
    ta, tw, to = dtypes
    a, w = torch.randn(T, H, k + 5).to(ta), torch.randn(H, n, k).to(tw)
    out = torch.full((T, H, n + 3), 7.0, dtype=to, device=dev)
    ops.heads_gemm(a.to(dev), w.to(dev), out, k=k, n=n)
    want = torch.einsum("thk,hnk->thn", a[..., :k].double(), w.double())
    tol = 1e-5 if to == torch.float32 else 3e-2
    assert torch.allclose(out[..., :n].cpu().double(), want, atol=tol * 5, rtol=tol)
    assert float(out[..., n:].float().min()) == 7.0
