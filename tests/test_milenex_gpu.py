"""Milenex on the GPU against the plain implementation (tests/plain_milenex.py, float64): every mechanism's kernels
alone -- with inputs made so that one key, one edge of a window, a sink or one expert decides the result --, then whole
models: prompts whole, decoded token by token, in portions down to two tokens, unequal requests in one batch, pages and
state slots that are used again, long decoding, greedy generation through the entry point and the scheduler -- in 32-bit
and in bfloat16, on configurations that differ in every size (tests/milenex_models.py).

In bfloat16 the whole models run with routers that have nothing to choose (every expert used, weighed by its score):
where a choice is a close call a rounding turns it, and the rows behind it are then another model's.  The choice itself
is tested on the routing kernel alone, and in 32-bit on the whole models."""
import math
import types

import numpy as np
import pytest
import torch

import helpers
import milenex_models
import plain_milenex as plain

pytestmark = pytest.mark.gpu

# A row of logits may differ from the plain row by this fraction of the plain row's root mean square (the errors' root
# mean square over the vocabulary), and no single logit by more than ten times that.
ROW_RMS = {"float32": 2e-5, "bfloat16": 6e-2}
LENGTHS = {"A": [1, 2, 9, 70, 150], "B": [3, 33, 64, 129], "C": [1, 17, 140], "D": [2, 66, 131, 200], "E": [1, 2, 3, 65, 190]}
CLOSE_CALL = 1e-5       # a 32-bit run is held to the plain rows up to a request's first routing margin below this


def close_rows(got, where, plain_logits, dtype, label, factor=1.0, upto=None):
    assert set(got) == set(where), f"{label}: rows produced {len(got)}, rows expected {len(where)}"
    limit, worst = ROW_RMS[dtype] * factor, 0.0
    for key in sorted(where):
        rid, pos = where[key]
        if upto is not None and pos >= upto.get(rid.replace("again", ""), 1 << 30):
            continue
        ref, row = plain_logits[rid][pos], got[key]
        assert np.all(np.isfinite(row)), f"{label}: non-finite logits at step {key[0]}, request {rid}, position {pos}"
        err, size = row - ref, float(np.sqrt(np.mean(ref * ref)))
        rms = float(np.sqrt(np.mean(err * err))) / size
        assert rms <= limit and float(np.abs(err).max()) <= 10 * limit * size, (
            f"{label}: first wrong row at step {key[0]}, request {rid}, position {pos}: errors' rms {rms:.3g} of the "
            f"row's (limit {limit:.3g}), largest {np.abs(err).max():.3g} of {size:.3g}")
        worst = max(worst, rms)
    return worst


def first_close_call(model) -> int:
    margins = model.closest_call()
    if margins is None:
        return 1 << 30
    near = torch.nonzero(margins < CLOSE_CALL)
    return int(near[0]) if len(near) else 1 << 30


def folder_for(tmp, name, dtype):
    if dtype == "bfloat16":
        return milenex_models.write_folder(tmp, name, dtype, config=milenex_models.every_expert(milenex_models.CONFIGS[name]),
                                           seed=milenex_models.SEEDS[name], tag="_every")
    return milenex_models.write_folder(tmp, name, dtype)


@pytest.fixture(scope="module")
def setups(tmp_path_factory):
    """(name, dtype) -> (folder, requests, plain logits of every request, first close call of every request)."""
    tmp, made = tmp_path_factory.mktemp("milenex"), {}

    def get(name, dtype):
        key = (name, dtype)
        if key not in made:
            folder = folder_for(tmp, name, dtype)
            model = plain.PlainMilenex(folder)
            requests = {f"r{i}": helpers.random_ids(n, model.cfg["vocab"], 700 + i) for i, n in enumerate(LENGTHS[name])}
            logits, upto = {}, {}
            for rid, ids in requests.items():
                logits[rid] = model.forward(ids).numpy()
                upto[rid] = first_close_call(model)
            made[key] = (folder, requests, logits, upto)
        return made[key]
    return get


def executor(folder, dtype, num_pages, page_tokens, max_requests=4, max_tokens=0, **kw):
    from bare_cuda_4gib_amd.engine import Executor, load_model
    model, _ = load_model(folder, dtype, "cuda:0")
    ex = Executor(model, num_pages=num_pages, max_requests=max_requests, max_tokens=max_tokens or num_pages * page_tokens,
                  page_tokens=page_tokens, poison=True, **kw)
    ex.cache.shuffle_free_pages(5)
    return ex


CASES = [(n, d) for n in sorted(milenex_models.CONFIGS) for d in ("float32", "bfloat16")]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompts(setups, name, dtype):
    folder, requests, logits, upto = setups(name, dtype)
    steps, where = helpers.trace_whole(requests)
    got = helpers.replay_in_process(executor(folder, dtype, 20, 16), steps)
    close_rows(got, where, logits, dtype, f"whole {name} {dtype}", upto=upto)


@pytest.mark.parametrize("name", sorted(milenex_models.CONFIGS))
def test_the_stream_after_every_layer_run(setups, name):
    """The residual stream behind every layer run (a looped layer counts each time) against the plain one, in 32-bit."""
    from bare_cuda_4gib_amd.engine import StepEntry
    folder, requests, _, upto = setups(name, "float32")
    rid = max(requests, key=lambda r: len(requests[r]))
    ids = requests[rid]
    model = plain.PlainMilenex(folder)
    _, after = model.forward(ids, return_layers=True)
    ex = executor(folder, "float32", 20, 16)
    seen = []
    for layer in ex.model.layers:         # a looped layer is one object that runs once a pass

        def run(x, ctx, cache, writes=True, _forward=layer.forward):
            _forward(x, ctx, cache, writes)
            seen.append(x.detach().float().cpu().double().clone())
        layer.forward = run
    ex.admit(rid)
    ex.step([StepEntry(rid, ids, [len(ids) - 1])])
    assert len(seen) == len(after) == len(model.order())
    rows = min(len(ids), upto[rid])
    for run, (mine, theirs) in enumerate(zip(seen, after)):
        size = float(theirs[:rows].pow(2).mean().sqrt())
        assert float((mine[:rows] - theirs[:rows]).abs().max()) <= 2e-4 * size, f"{name}: layer run {run}"


@pytest.mark.parametrize("name,dtype", CASES)
def test_prefill_against_decoding_token_by_token(setups, name, dtype):
    """Most of a request in one step, its last 75 tokens one by one: every window (up to 70 keys) passes over decoded
    tokens, the convolutions' and the shift's states move once a step."""
    folder, requests, logits, upto = setups(name, dtype)
    steps, where = helpers.trace_tail_one_by_one(requests, tail=75)
    got = helpers.replay_in_process(executor(folder, dtype, 20, 16), steps)
    close_rows(got, where, logits, dtype, f"tail {name} {dtype}", upto=upto)


@pytest.mark.parametrize("name,dtype", CASES)
def test_portions_down_to_two_tokens(setups, name, dtype):
    folder, requests, logits, upto = setups(name, dtype)
    for seed, sizes in ((1, (17, 2, 5, 64, 3, 2, 31, 9)), (2, (2, 2, 3, 16, 15, 1, 33, 70))):
        steps, where = helpers.trace_portions(requests, seed, sizes)
        got = helpers.replay_in_process(executor(folder, dtype, 20, 16), steps)
        close_rows(got, where, logits, dtype, f"portions {name} {dtype} {seed}", upto=upto)


@pytest.mark.parametrize("name,dtype", CASES)
def test_mixed_batches_with_pages_and_slots_used_again(setups, name, dtype):
    """Up to three live requests in three state slots and a pool just large enough: portions beside decoded tokens,
    requests left out of steps, pages and slots handed to the next request without being cleared by anyone but the
    admission (unowned pages hold NaN)."""
    folder, requests, logits, upto = setups(name, dtype)
    many = dict(requests)
    many.update({rid + "again": ids for rid, ids in requests.items()})            # the same requests once more, in other slots
    plain_logits = dict(logits)
    plain_logits.update({rid + "again": logits[rid] for rid in requests})
    for seed in (3, 4):
        steps, where, peak = helpers.trace_mixed(many, seed, max_live=3, tail=10, page_tokens=16)
        ex = executor(folder, dtype, peak // 16, 16, max_requests=3, max_tokens=208)
        got = helpers.replay_in_process(ex, steps)
        close_rows(got, where, plain_logits, dtype, f"mixed {name} {dtype} {seed}", upto=upto)
        assert ex.cache.pages_in_use() == 0 and ex.cache.free_slots == 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_in_one_batch_against_each_alone(setups, dtype):
    from bare_cuda_4gib_amd.engine import StepEntry
    folder, requests, _, _ = setups("A", dtype)
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


@pytest.mark.parametrize("name", ["A", "D"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_the_first_tokens(setups, name, dtype):
    """Two tokens, then 300 one by one over pages of 16: the shift and the convolutions from the very first tokens, the
    rotations and the windows far from the start, pages the windows have left."""
    from bare_cuda_4gib_amd.engine import StepEntry
    folder, _, _, _ = setups(name, dtype)
    model = plain.PlainMilenex(folder)
    ids = helpers.random_ids(302, model.cfg["vocab"], 9)
    want = model.forward(ids).numpy()
    upto = {"r": first_close_call(model)}
    ex = executor(folder, dtype, 19, 16, max_requests=2)
    ex.admit("r")
    got = {}
    rows = ex.step([StepEntry("r", ids[:2], [0, 1])]).cpu().numpy()
    got[(0, 0)], got[(0, 1)] = rows[0], rows[1]
    for p in range(2, len(ids)):
        got[(0, p)] = ex.step([StepEntry("r", [ids[p]], [0])]).cpu().numpy()[0]
    where = {(0, p): ("r", p) for p in range(len(ids))}
    close_rows(got, where, {"r": want}, dtype, f"long decoding {name} {dtype}", upto=upto)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point_and_the_scheduler(setups, dtype):
    from bare_cuda_4gib_amd.engine import Engine, generate_batch
    folder, _, _, _ = setups("A", dtype)
    model = plain.PlainMilenex(folder)
    prompts = [helpers.random_ids(n, model.cfg["vocab"], 50 + n) for n in (1, 5, 21, 40)]
    engine = Engine(folder, max_tokens=96, max_seqs=3, dtype=dtype, page_tokens=16, prefill_chunk=16)   # four requests, three slots
    together = generate_batch(engine, prompts, 24)
    margin = 1e-4 if dtype == "float32" else 0.3
    for prompt, tokens in zip(prompts, together):
        assert len(tokens) == 24
        full = model.forward(list(prompt) + list(tokens)).numpy()
        turned = first_close_call(model)
        for i, tok in enumerate(tokens):                # every chosen token is the plain best, or within a near-tie of it
            if len(prompt) - 1 + i >= turned:
                break
            row = full[len(prompt) - 1 + i]
            assert float(row.max() - row[tok]) <= margin, f"token {i} ({tok}) lies {row.max() - row[tok]:.4g} below the plain best"
    stats = engine.stats()
    assert stats["kv_pages_used"] == 0 and stats["running"] == 0


def test_the_command_line_generates_from_a_folder(setups):
    """bin/llm-infer over a Milenex folder: the architecture is chosen by config.json, ids in, ids out."""
    import os
    import subprocess
    import sys
    folder, _, _, _ = setups("B", "float32")
    model = plain.PlainMilenex(folder)
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
    folder, requests, logits, upto = setups("A", "float32")
    steps, where, peak = helpers.trace_mixed(requests, 8, max_live=4, tail=6, page_tokens=64)
    got = helpers.replay_subprocess(folder, "float32", steps, str(tmp_path / "out"), peak, milenex_models.CONFIGS["A"]["vocab"])
    close_rows(got, where, logits, "float32", "bin/trace_run", upto=upto)


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
@pytest.mark.parametrize("channels", [37, 64])
def test_norm_with_a_weight_around_zero(dtype, channels):
    from bare_cuda_4gib_amd.engine.spec import PartSpec
    from bare_cuda_4gib_amd.parts import build_part
    torch.manual_seed(channels)
    x, g = torch.randn(9, channels) * 3.0, (torch.randn(channels) * 0.3).to(dtype)
    part = build_part("norm", PartSpec("rmsnorm", dict(size=channels, eps=1e-3, offset=1.0)))
    part.bind({"weight": g.to(DEV)}, types.SimpleNamespace(act_dtype=dtype, device=DEV))
    got = part.forward(x.to(DEV)).float().cpu().double()
    want = plain.zero_centred_norm(x.double(), g.double(), 1e-3)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert torch.allclose(got, want, atol=tol, rtol=tol)
    assert float((want - plain.unit_rms(x.double(), 1e-3) * g.double()).abs().max()) > 0.5         # (the one counts)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [2, 3, 5])
def test_shift_and_convolution_over_portions_and_slots_used_again(dtype, taps):
    """Three requests of unequal length cut into unequal portions that share steps, down to one row, shorter than the
    taps at the very start; their states lie in slots given in another order, and a slot is used again by a new request
    without being cleared by anyone but its first portion (cached 0).  Against the plain functions on whole sequences."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(taps)
    C = 44
    seqs = [torch.randn(n, C).to(dtype) for n in (23, 9, 1, 14)]
    conv_w, shift_m = torch.randn(C, taps), torch.rand(C)
    want_conv = [plain.short_convolution(s.double(), conv_w.double()) for s in seqs]
    want_shift = [plain.token_shift(s.double(), shift_m.double()) for s in seqs]
    tails = torch.full((3, taps - 1, C), float("nan"), dtype=dtype, device=DEV)
    last = torch.full((3, 1, C), float("nan"), dtype=dtype, device=DEV)
    w_taps = conv_w.t().contiguous().to(DEV)
    w_shift = torch.stack([shift_m, -shift_m], dim=0).contiguous().to(DEV)
    # (request, slot, portions): request 3 takes request 1's slot after it has ended
    plan = [[(0, 2, 1), (1, 0, 4)], [(0, 2, 2), (1, 0, 5), (2, 1, 1)], [(0, 2, 7)], [(0, 2, 1), (3, 0, 1)], [(0, 2, 12), (3, 0, 13)]]
    done = [0, 0, 0, 0]
    got_conv, got_shift = [[] for _ in seqs], [[] for _ in seqs]
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    for step in plan:
        ctx = step_context([n for _, _, n in step], [done[r] for r, _, _ in step], [slot for _, slot, _ in step])
        x = torch.cat([seqs[r][done[r]:done[r] + n] for r, _, n in step]).to(DEV)
        wide = torch.cat([torch.zeros(x.shape[0], 3, dtype=dtype, device=DEV), x], dim=1)      # a part of wider rows
        if done[step[0][0]] == 0 or any(done[r] == 0 for r, _, _ in step):
            for r, slot, _ in step:
                if done[r] == 0:
                    tails[slot].zero_()
                    last[slot].zero_()
        y = ops.causal_conv(wide[:, 3:], w_taps, tails, ctx).float().cpu().double()
        z = ops.causal_conv(x, w_shift, last, ctx, add_input=True).float().cpu().double()
        at = 0
        for r, _, n in step:
            got_conv[r].append(y[at:at + n])
            got_shift[r].append(z[at:at + n])
            at, done[r] = at + n, done[r] + n
    for r in range(len(seqs)):
        assert done[r] == len(seqs[r])
        assert torch.allclose(torch.cat(got_conv[r]), want_conv[r], atol=tol, rtol=tol), r
        assert torch.allclose(torch.cat(got_shift[r]), want_shift[r], atol=tol, rtol=tol), r


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C", [44, 320, 2500])
def test_norm_and_shift_in_one_pass_over_portions_and_slots_used_again(dtype, C):
    """The norm with a weight around zero and the token shift behind it as one kernel: requests cut into unequal portions
    that share steps, states in slots given in another order, a slot used again by a new request; against the plain
    functions on whole sequences, and against the two kernels one after the other."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(C)
    eps = 1e-3
    seqs = [torch.randn(n, C) * 2.0 for n in (23, 9, 1, 14)]
    g, m = (torch.randn(C) * 0.3), torch.rand(C)
    want = [plain.token_shift(plain.zero_centred_norm(s.double(), g.double(), eps).to(dtype).double(), m.double()) for s in seqs]
    state = torch.full((3, 1, C), float("nan"), dtype=dtype, device=DEV)
    apart = torch.full((3, 1, C), float("nan"), dtype=dtype, device=DEV)
    w, mix = (1.0 + g).to(DEV), m.to(DEV)
    taps = torch.stack([m, -m], dim=0).contiguous().to(DEV)
    plan = [[(0, 2, 1), (1, 0, 4)], [(0, 2, 2), (1, 0, 5), (2, 1, 1)], [(0, 2, 7)], [(0, 2, 1), (3, 0, 1)], [(0, 2, 12), (3, 0, 13)]]
    done, got = [0, 0, 0, 0], [[] for _ in seqs]
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    for step in plan:
        ctx = step_context([n for _, _, n in step], [done[r] for r, _, _ in step], [slot for _, slot, _ in step])
        x = torch.cat([seqs[r][done[r]:done[r] + n] for r, _, n in step]).to(DEV)
        for r, slot, _ in step:
            if done[r] == 0:
                state[slot].zero_()
                apart[slot].zero_()
        y = ops.rmsnorm_shift(x, w, eps, mix, state, ctx, dtype)
        two = ops.causal_conv(ops.rmsnorm(x, w, eps, dtype), taps, apart, ctx, add_input=True)
        assert torch.allclose(y.float(), two.float(), atol=tol, rtol=tol)
        at = 0
        for r, _, n in step:
            got[r].append(y[at:at + n].float().cpu().double())
            at, done[r] = at + n, done[r] + n
    assert torch.allclose(state.float().nan_to_num(7.0), apart.float().nan_to_num(7.0), atol=tol, rtol=tol)       # the same states
    for r in range(len(seqs)):
        assert torch.allclose(torch.cat(got[r]), want[r], atol=tol, rtol=tol), r


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,dims,base", [(3, 8, 8, 10000.0), (2, 48, 24, 500.0), (5, 7, 6, 30.0), (1, 130, 2, 7.0), (4, 10, 0, 1.0)])
def test_neighbours_are_rotated_then_the_head_is_divided_by_its_root_mean_square(dtype, heads, dim, dims, base):
    from bare_cuda_4gib_amd.csrc import ops
    from bare_cuda_4gib_amd.engine.spec import PartSpec
    from bare_cuda_4gib_amd.parts import build_part
    torch.manual_seed(dim)
    T, P, eps = 6, 4, 1e-2
    wide = (torch.randn(T, heads * dim + 11) * 0.2).to(dtype)         # (small: the eps inside the root counts)
    x = wide[:, 5:5 + heads * dim]
    positions = torch.tensor([0, 1, 2, 1000, 70001, 3], dtype=torch.int32)
    table = None
    if dims:
        part = build_part("position", PartSpec("rotary", dict(theta=base, dim=dims, pairing="neighbours")))
        ctx = types.SimpleNamespace(positions=positions.to(DEV), shared=lambda key, make: make())
        table = part.table(ctx)
        assert part.neighbours
    want = plain.unit_rms(plain.neighbour_rotation(x.double().view(T, heads, dim), positions, dims, base), eps)
    out = torch.zeros(T, heads, dim, device=DEV)
    ops.heads_prepare(wide.to(DEV)[:, 5:5 + heads * dim], heads, dim, out, table=table, neighbours=True, unit_after=True, eps=eps)
    assert torch.allclose(out.cpu().double(), want, atol=3e-5, rtol=3e-5)
    if dims >= 6:      # (neither the other pairing nor the norm before the rotation's place would pass)
        halves = x.double().view(T, heads, dim).clone()
        a, b = halves[..., :dims // 2].clone(), halves[..., dims // 2:dims].clone()
        i = torch.arange(dims // 2, dtype=torch.float64)
        ang = positions.double()[:, None] * base ** (-2.0 * i / dims)[None, :]
        halves[..., :dims // 2] = a * torch.cos(ang)[:, None] - b * torch.sin(ang)[:, None]
        halves[..., dims // 2:dims] = b * torch.cos(ang)[:, None] + a * torch.sin(ang)[:, None]
        assert float((plain.unit_rms(halves, eps) - want).abs().max()) > 0.1
    slot_map = torch.tensor([9, 2, 0, 7, 5, 11], dtype=torch.int32)
    cache = torch.zeros(3, heads, P, dim, dtype=dtype, device=DEV)
    ops.heads_prepare(wide.to(DEV)[:, 5:5 + heads * dim], heads, dim, cache, table=table, slot_map=slot_map.to(DEV), page_tokens=P,
                      neighbours=True, unit_after=True, eps=eps)
    tol = 3e-5 if dtype == torch.float32 else 1e-2
    flat = cache.cpu().double().permute(0, 2, 1, 3).reshape(3 * P, heads, dim)
    for t in range(T):
        assert torch.allclose(flat[slot_map[t]], want[t], atol=tol, rtol=tol), t


def paged(rows_k, rows_v, pages, P, dtype, n_pages):
    """Caches [pages, heads, P, size] that hold NaN but for the given rows, laid into the given pages."""
    k = torch.full((n_pages, rows_k.shape[1], P, rows_k.shape[2]), float("nan"), dtype=dtype, device=DEV)
    v = torch.full((n_pages, rows_v.shape[1], P, rows_v.shape[2]), float("nan"), dtype=dtype, device=DEV)
    for j in range(rows_k.shape[0]):
        k[pages[j // P], :, j % P] = rows_k[j].to(dtype).to(DEV)
        v[pages[j // P], :, j % P] = rows_v[j].to(dtype).to(DEV)
    return k, v


def plain_heads(q, keys, values, pos, G, scale, window, sink, far=None, talk=None, gate=None):
    """The plain result for one row at position ``pos`` (the last of pos + 1 tokens): q [H, d], keys [n, G, d], values
    [n, G, e] -> ([H, e], weights [H, pos + 1]).  Uses the plain weights of whole sequences: only the last row's count."""
    H, n = q.shape[0], pos + 1
    weights = []
    for a in range(H):
        g = a // (H // G)
        qs = torch.zeros(n, q.shape[1], dtype=torch.float64)
        qs[-1] = q[a].double()
        r1, r2 = (float(far[0][a]), float(far[1][a])) if far is not None else (0.0, 0.0)
        weights.append(plain.window_weights(qs, keys[:n, g].double(), scale, window if window > 0 else n, float(sink[a]), r1, r2)[-1])
    weights = torch.stack(weights)
    mixed = talk.double() @ weights if talk is not None else weights
    out = torch.stack([mixed[a] @ values[:n, a // (H // G)].double() for a in range(H)])
    if gate is not None:
        out = out * torch.sigmoid(gate.double())[:, None]
    return out, weights


def run_heads(kind, q_rows, k_cache, v_cache, table, ctx, H, G, d, e, window, scale, sink, far, talk, gate, parts=0, keep=None):
    from bare_cuda_4gib_amd.csrc import ops
    dev = lambda t: t.to(DEV) if t is not None else None      # noqa: E731
    far = (dev(far[0].float()), dev(far[1].float())) if far is not None else None
    if kind == "own":
        t = q_rows.shape[0]
        return ops.attention_maps(q_rows.view(t, H, 1, d).contiguous().to(DEV), k_cache, v_cache, table, ctx, torch.float32, H, G, 1, d, e,
                                  window, 0, scale, sink=dev(sink.float()), far=far).cpu().double()
    return ops.attention_talk(q_rows.contiguous().to(DEV), k_cache, v_cache, table, ctx, torch.float32, H, G, d, e, window, scale,
                              sink=dev(sink.float()), far=far, talk=dev(talk.float()) if talk is not None else None,
                              gate=dev(gate), parts=parts, keep_scores=keep).cpu().double()


SIZES = [(4, 2, 12, 20), (3, 3, 10, 70), (6, 1, 44, 100), (2, 1, 7, 130), (2, 2, 72, 200), (12, 4, 6, 9), (18, 6, 8, 12)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["own", "mixed"])
@pytest.mark.parametrize("sizes", SIZES)
@pytest.mark.parametrize("needle", [0, 7, 8, 63, 64, 120, 199])
def test_attention_finds_one_key_among_hundreds(dtype, kind, needle, sizes):
    """200 cached keys in scattered pages of 8, no window; one key, far back, at a page's border or the row's own, is
    made to score far above the others (and above the sink and the distance's penalty) in one head: that head's weight
    goes there, the result equals the plain one for every head -- with every head's own weights (``own``) and with weights
    mixed among the heads and a gate on each (``mixed``).  As a decoded token and as the last rows of a portion."""
    torch.manual_seed(needle)
    (H, G, d, e), n, P, scale = sizes, 200, 8, 0.3
    keys, values = (torch.randn(n, G, d) * 0.3).to(dtype).float(), torch.randn(n, G, e).to(dtype).float()
    q = torch.randn(H, d)
    sink = torch.randn(H) + 1.0
    far = (torch.rand(H) * 0.5 + 0.2, torch.rand(H) * 2.0 + 0.1)
    talk = torch.eye(H) * 0.8 + torch.randn(H, H) * 0.25 if kind == "mixed" else None
    mark = min(1, H - 1)
    keys[needle, mark // (H // G)] = (q[mark] / float(q[mark] @ q[mark]) * 20.0 / scale).to(dtype).float()
    pages = torch.randperm(40)[:n // P]
    k_cache, v_cache = paged(keys, values, pages, P, dtype, 40)
    table = pages.to(torch.int32).view(1, -1).to(DEV)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for lengths, cached in (([1], [n - 1]), ([6], [n - 6])):
        ctx = step_context(lengths, cached, [0])
        qs = q.view(1, H, d).repeat(lengths[0], 1, 1)
        gate = torch.randn(lengths[0], H) if kind == "mixed" else None
        got = run_heads(kind, qs, k_cache, v_cache, table, ctx, H, G, d, e, 0, scale, sink, far, talk,
                        gate.to(dtype) if gate is not None else None)
        for r in range(lengths[0]):
            pos = cached[0] + r
            want, weights = plain_heads(q, keys, values, pos, G, scale, 0, sink, far, talk,
                                        gate[r].to(dtype) if gate is not None else None)
            assert torch.allclose(got[r].view(H, e), want, atol=tol * max(1.0, float(want.abs().max())), rtol=tol), (needle, pos)
            if needle <= pos:
                assert float(weights[mark][needle]) > 0.9


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("parts", [1, 2, 3, 5, 64])
@pytest.mark.parametrize("window", [0, 100, 64])
@pytest.mark.parametrize("keep", [True, False])
@pytest.mark.parametrize("H,G", [(6, 2), (18, 6), (20, 1)])
def test_mixed_heads_with_a_row_s_keys_cut_into_parts(dtype, parts, window, keep, H, G):
    """The keys of every row cut into one to 64 parts (more parts than tiles of keys: the last are empty), a needle in the
    last part's tile, rows of unequal reach in one step: the parts' statistics and outputs add up to the plain result,
    with the first walk's scores kept for the second and without; with more heads than a workgroup has waves the kept
    scores let the heads be cut over workgroups too."""
    torch.manual_seed(parts)
    d, e, n, P, scale = 24, 36, 300, 16, 0.3
    keys, values = (torch.randn(n, G, d) * 0.3).to(dtype).float(), torch.randn(n, G, e).to(dtype).float()
    q = torch.randn(H, d)
    sink, far = torch.randn(H) + 1.0, (torch.rand(H) * 0.5 + 0.2, torch.rand(H) * 2.0 + 0.1)
    talk = torch.eye(H) * 0.8 + torch.randn(H, H) * 0.25
    keys[n - 3, 4 // (H // G)] = (q[4] / float(q[4] @ q[4]) * 20.0 / scale).to(dtype).float()
    pages = torch.randperm(30)[:-(-n // P)]
    k_cache, v_cache = paged(keys, values, pages, P, dtype, 30)
    table = pages.to(torch.int32).view(1, -1).repeat(2, 1).to(DEV)         # two requests over the same pages
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    lengths, cached = [3, 1], [n - 3, 40]
    ctx = step_context(lengths, cached, [0, 1])
    gate = torch.randn(4, H)
    got = run_heads("mixed", q.view(1, H, d).repeat(4, 1, 1), k_cache, v_cache, table, ctx, H, G, d, e, window, scale, sink, far, talk,
                    gate, parts=parts, keep=keep)
    for r, pos in enumerate([n - 3, n - 2, n - 1, 40]):
        want, weights = plain_heads(q, keys, values, pos, G, scale, window, sink, far, talk, gate[r])
        assert torch.allclose(got[r].view(H, e), want, atol=tol * max(1.0, float(want.abs().max())), rtol=tol), (parts, pos)
        if pos >= n - 3:
            assert float(weights[4][n - 3]) > 0.9


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["own", "mixed"])
@pytest.mark.parametrize("window", [1, 6, 9, 50, 63, 64, 65, 96, 130])
@pytest.mark.parametrize("where", ["window_in", "window_out"])
def test_attention_at_the_edges_of_the_window(dtype, kind, window, where):
    """A key made to stand out just inside the window takes the weight; the same key one place further back is not seen
    at all, and with nothing else in sight the sink takes what is left -- as a decoded token and in a portion whose rows'
    windows begin at different keys, over pages of 16."""
    torch.manual_seed(window)
    H, G, d, e, n, P, scale = 4, 2, 12, 20, 150, 16, 0.3
    keys, values = (torch.randn(n, G, d) * 0.3).to(dtype).float(), torch.randn(n, G, e).to(dtype).float()
    q = torch.randn(H, d)
    sink, far = torch.randn(H) + 1.0, (torch.rand(H) * 0.5 + 0.2, torch.rand(H) * 2.0 + 0.1)
    talk = torch.eye(H) * 0.8 + torch.randn(H, H) * 0.25 if kind == "mixed" else None
    pos_last = n - 1
    needle = pos_last - window + 1 if where == "window_in" else pos_last - window
    keys[needle, 0] = (q[0] / float(q[0] @ q[0]) * 20.0 / scale).to(dtype).float()        # (head 0 reads key/value head 0)
    pages = torch.randperm(20)[:-(-n // P)]
    k_cache, v_cache = paged(keys, values, pages, P, dtype, 20)
    table = pages.to(torch.int32).view(1, -1).to(DEV)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for lengths, cached in (([1], [n - 1]), ([5], [n - 5])):
        ctx = step_context(lengths, cached, [0])
        qs = q.view(1, H, d).repeat(lengths[0], 1, 1)
        gate = torch.randn(lengths[0], H) if kind == "mixed" else None
        got = run_heads(kind, qs, k_cache, v_cache, table, ctx, H, G, d, e, window, scale, sink, far, talk, gate)
        for r in range(lengths[0]):
            pos = cached[0] + r
            want, weights = plain_heads(q, keys, values, pos, G, scale, window, sink, far, talk, gate[r] if gate is not None else None)
            assert torch.allclose(got[r].view(H, e), want, atol=tol * max(1.0, float(want.abs().max())), rtol=tol), (where, pos)
            if pos == pos_last:
                if where == "window_in":
                    assert float(weights[0][needle]) > 0.9
                else:
                    assert float(weights[0][needle]) == 0.0 and float(weights[0].sum()) < 0.999      # (the sink's share)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["own", "mixed"])
def test_attention_of_the_first_tokens_a_large_sink_and_unequal_requests(dtype, kind):
    """Three requests in one step -- the first token of a sequence, a portion from position 0, a decoded token far in --
    each with a block table of its own; one head's sink is so large that the head gives next to nothing, another's so
    small that it does not count."""
    torch.manual_seed(8)
    H, G, d, e, P, scale, window = 3, 3, 10, 6, 4, 0.5, 5
    lengths, cached = [1, 9, 1], [0, 0, 30]
    n_pages = 24
    k_cache = torch.full((n_pages + 1, G, P, d), float("nan"), dtype=dtype, device=DEV)
    v_cache = torch.full((n_pages + 1, G, P, e), float("nan"), dtype=dtype, device=DEV)
    perm = torch.randperm(n_pages)
    tables, seqs, at = torch.full((3, 8), -1, dtype=torch.int32), [], 0
    for s, (new, old) in enumerate(zip(lengths, cached)):
        n = new + old
        keys, values = torch.randn(n, G, d).to(dtype).float(), torch.randn(n, G, e).to(dtype).float()
        pages = perm[at:at + -(-n // P)]
        at += len(pages)
        tables[s, :len(pages)] = pages.to(torch.int32)
        for j in range(n):
            k_cache[pages[j // P], :, j % P] = keys[j].to(dtype).to(DEV)
            v_cache[pages[j // P], :, j % P] = values[j].to(dtype).to(DEV)
        seqs.append((keys, values))
    ctx = step_context(lengths, cached, [0, 1, 2])
    q = torch.randn(sum(lengths), H, d)
    sink = torch.tensor([12.0, -30.0, 0.3])
    far = (torch.rand(H) * 0.5 + 0.2, torch.rand(H) * 2.0 + 0.1) if kind == "mixed" else None
    talk = torch.eye(H) * 0.8 + torch.randn(H, H) * 0.25 if kind == "mixed" else None
    gate = torch.randn(sum(lengths), H).to(dtype) if kind == "mixed" else None
    got = run_heads(kind, q, k_cache, v_cache, tables.to(DEV), ctx, H, G, d, e, window, scale, sink, far, talk, gate)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    row = 0
    for s, (new, old) in enumerate(zip(lengths, cached)):
        for i in range(new):
            want, weights = plain_heads(q[row], seqs[s][0], seqs[s][1], old + i, G, scale, window, sink, far, talk,
                                        gate[row] if gate is not None else None)
            assert torch.allclose(got[row].view(H, e), want, atol=tol, rtol=tol), (s, i)
            assert float(weights[0].sum()) < 0.05 and float(weights[1].sum()) > 0.999999
            row += 1


@pytest.mark.parametrize("experts,top,groups,keep", [(8, 3, 4, 2), (6, 2, 3, 2), (5, 5, 1, 1), (4, 1, 1, 1), (3, 2, 1, 1), (64, 6, 8, 3),
                                                     (12, 3, 4, 1), (8, 8, 2, 2), (40, 7, 1, 1)])
def test_the_router_chooses_among_the_best_groups_and_weighs_by_the_plain_scores(experts, top, groups, keep):
    """Logits of many rows with corrections large enough to change the choice and negative enough that every choice score
    of a group lies below zero (a group left out must count as minus infinity, not as zero); rows whose choice is a
    close call in 32-bit are left out.  The logits are a part of wider rows."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(experts * 10 + top)
    T = 300
    wide = torch.randn(T, experts + 3) * 2.0
    correction = torch.randn(experts) * 0.2 - 1.3
    z = wide[:, :experts]
    chosen, weights = plain.route(z.double(), correction.double(), top, groups, keep)
    margin = plain.route_margin(z.double(), correction.double(), top, groups, keep)
    got_w, got_c = ops.moe_route(wide.to(DEV)[:, :experts], experts, top, groups, keep, correction.to(DEV), want_chosen=True)
    got_w, got_c = got_w.cpu().double(), got_c.cpu().long()
    want_w = torch.zeros(T, experts, dtype=torch.float64).scatter_(1, chosen, weights)
    sure = margin > 1e-5
    assert int(sure.sum()) > T * 0.9
    assert torch.allclose(got_w[sure], want_w[sure], atol=1e-6, rtol=1e-5)
    assert torch.equal(got_c[sure].sort(dim=1).values, chosen[sure].sort(dim=1).values)
    assert bool(((got_w > 0).sum(dim=1) == top).all())
    if keep < groups and top > keep:         # (the groups matter: without them other experts would win in some rows)
        free, _ = plain.route(z.double(), correction.double(), top, 1, 1)
        assert not torch.equal(free.sort(dim=1).values, chosen.sort(dim=1).values)
    if top < experts:         # (so does the correction)
        plain_choice, _ = plain.route(z.double(), torch.zeros(experts, dtype=torch.float64), top, groups, keep)
        assert not torch.equal(plain_choice.sort(dim=1).values, chosen.sort(dim=1).values)
    assert int(((torch.softmax(z.double(), -1) + correction.double()).max(dim=1).values < 0.0).sum()) > T // 2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,ff,shared_ff", [(3, 10, 7), (4, 16, 0), (1, 5, 3), (6, 24, 16), (0, 0, 12)])
def test_weighted_clamped_gated_units_and_the_shared_one(dtype, experts, ff, shared_ff):
    """Gates far above the limit stay at the limit, gates far below it are not clamped; ups are clamped on both sides;
    the shared unit has a limit of its own and a gate for every row."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(experts + ff)
    T, limit, shared_limit = 13, 0.8, 1.7
    gu = (torch.randn(T, 2 * (experts * ff + shared_ff)) * 2.0).to(dtype)
    weights = torch.rand(T, experts) * (torch.rand(T, experts) > 0.4) if experts else None
    logit = torch.randn(T, 4)
    got = ops.routed_glu(gu.to(DEV), weights.float().to(DEV) if experts else None, experts, ff, limit, shared_ff=shared_ff,
                         shared_limit=shared_limit, shared_logit=logit.to(DEV)[:, 2:3] if shared_ff else None).float().cpu().double()
    want = []
    for j in range(experts):
        part = gu[:, 2 * ff * j:2 * ff * (j + 1)].double()
        want.append(plain.clamped_glu(part[:, :ff], part[:, ff:], limit) * weights[:, j:j + 1].double())
    if shared_ff:
        part = gu[:, 2 * ff * experts:].double()
        want.append(plain.clamped_glu(part[:, :shared_ff], part[:, shared_ff:], shared_limit) * torch.sigmoid(logit[:, 2:3].double()))
    want = torch.cat(want, dim=1)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert got.shape == want.shape and torch.allclose(got, want, atol=tol, rtol=tol)
    assert float(gu.float().max()) > 2 * limit and float(gu.float().min()) < -2 * limit


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_exact_gelu(dtype):
    from bare_cuda_4gib_amd.csrc import ops
    z = torch.linspace(-9.0, 9.0, 1001).view(7, 143).to(dtype)
    got = ops.gelu(z.to(DEV)).float().cpu().double()
    want = plain.gelu_erf(z.double())
    assert torch.allclose(got, want, atol=2e-6 if dtype == torch.float32 else 2e-2, rtol=1e-5 if dtype == torch.float32 else 1e-2)
    tanh_form = 0.5 * z.double() * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z.double() + 0.044715 * z.double() ** 3)))
    if dtype == torch.float32:
        assert float((got - tanh_form).abs().max()) > 1e-4            # (the other gelu would not pass)
