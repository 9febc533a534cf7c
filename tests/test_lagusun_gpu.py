"""Lagusun on the GPU against the plain implementation (tests/plain_lagusun.py, float64): every mechanism's kernels
alone -- with inputs made so that one key, one edge of a block or a window, the one in the denominator or one expert
decides the result --, then whole models: prompts whole, decoded token by token, in portions down to two tokens,
unequal requests in one batch, pages and slots that are used again, long decoding, greedy generation through the entry
point and the scheduler -- in 32-bit and in bfloat16, on configurations that differ in every size
(tests/lagusun_models.py).

In bfloat16 the whole models run with routers that have nothing to choose (every expert used, weighed by its score):
where a choice is a close call a rounding turns it, and the rows behind it are then another model's.  The choice itself
is tested on the routing kernel alone, and in 32-bit on the whole models."""
import math
import types

import numpy as np
import pytest
import torch

import helpers
import lagusun_models
import plain_lagusun as plain

pytestmark = pytest.mark.gpu

# A row of logits may differ from the plain row by this fraction of the plain row's root mean square (the errors' root
# mean square over the vocabulary), and no single logit by more than ten times that.
ROW_RMS = {"float32": 2e-5, "bfloat16": 6e-2}
LENGTHS = {"A": [1, 2, 9, 70, 150], "B": [3, 33, 64, 141], "C": [1, 17, 140], "D": [2, 66, 131, 200], "E": [1, 2, 3, 65, 190],
           "F": [1, 5, 101, 130], "G": [5, 150, 260]}
CLOSE_CALL = 1e-5       # a 32-bit run is held to the plain rows up to a request's first routing margin below this
DEV = "cuda:0"


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
        return lagusun_models.write_folder(tmp, name, dtype, config=lagusun_models.every_expert(lagusun_models.CONFIGS[name]),
                                           seed=lagusun_models.SEEDS[name], tag="_every")
    return lagusun_models.write_folder(tmp, name, dtype)


@pytest.fixture(scope="module")
def setups(tmp_path_factory):
    """(name, dtype) -> (folder, requests, plain logits of every request, first close call of every request)."""
    tmp, made = tmp_path_factory.mktemp("lagusun"), {}

    def get(name, dtype):
        key = (name, dtype)
        if key not in made:
            folder = folder_for(tmp, name, dtype)
            model = plain.PlainLagusun(folder)
            requests = {f"r{i}": helpers.random_ids(n, model.cfg["vocab"], 900 + i) for i, n in enumerate(LENGTHS[name])}
            logits, upto = {}, {}
            for rid, ids in requests.items():
                logits[rid] = model.forward(ids).numpy()
                upto[rid] = first_close_call(model)
            made[key] = (folder, requests, logits, upto)
        return made[key]
    return get


def executor(folder, dtype, num_pages, page_tokens, max_requests=4, max_tokens=0, **kw):
    from bare_cuda_4gib_amd.engine import Executor, load_model
    model, _ = load_model(folder, dtype, DEV)
    ex = Executor(model, num_pages=num_pages, max_requests=max_requests, max_tokens=max_tokens or num_pages * page_tokens,
                  page_tokens=page_tokens, poison=True, **kw)
    ex.cache.shuffle_free_pages(5)
    return ex


CASES = [(n, d) for n in sorted(lagusun_models.CONFIGS) for d in ("float32", "bfloat16")]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompts(setups, name, dtype):
    folder, requests, logits, upto = setups(name, dtype)
    steps, where = helpers.trace_whole(requests)
    got = helpers.replay_in_process(executor(folder, dtype, 40, 16), steps)
    close_rows(got, where, logits, dtype, f"whole {name} {dtype}", upto=upto)


@pytest.mark.parametrize("name", sorted(lagusun_models.CONFIGS))
def test_the_stream_after_every_layer_run(setups, name):
    """The residual stream behind every layer run (a looped layer counts each time) against the plain one, in 32-bit."""
    from bare_cuda_4gib_amd.engine import StepEntry
    folder, requests, _, upto = setups(name, "float32")
    rid = max(requests, key=lambda r: len(requests[r]))
    ids = requests[rid]
    model = plain.PlainLagusun(folder)
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
    assert len(seen) == len(after) == len(model.runs())
    rows = min(len(ids), upto[rid])
    for run, (mine, theirs) in enumerate(zip(seen, after)):
        size = float(theirs[:rows].pow(2).mean().sqrt())
        assert float((mine[:rows] - theirs[:rows]).abs().max()) <= 2e-4 * size, f"{name}: layer run {run}"


@pytest.mark.parametrize("name,dtype", CASES)
def test_prefill_against_decoding_token_by_token(setups, name, dtype):
    """Most of a request in one step, its last 75 tokens one by one: every window and block (up to 70 keys) passes over
    decoded tokens."""
    folder, requests, logits, upto = setups(name, dtype)
    steps, where = helpers.trace_tail_one_by_one(requests, tail=75)
    got = helpers.replay_in_process(executor(folder, dtype, 20, 16), steps)
    close_rows(got, where, logits, dtype, f"tail {name} {dtype}", upto=upto)


@pytest.mark.parametrize("name,dtype", CASES)
def test_portions_down_to_two_tokens(setups, name, dtype):
    """Portions are cut in the middle of pages, windows and blocks: a block counts from the sequence's first token."""
    folder, requests, logits, upto = setups(name, dtype)
    for seed, sizes in ((1, (17, 2, 5, 64, 3, 2, 31, 9)), (2, (2, 2, 3, 16, 15, 1, 33, 70))):
        steps, where = helpers.trace_portions(requests, seed, sizes)
        got = helpers.replay_in_process(executor(folder, dtype, 20, 16), steps)
        close_rows(got, where, logits, dtype, f"portions {name} {dtype} {seed}", upto=upto)


@pytest.mark.parametrize("name,dtype", CASES)
def test_mixed_batches_with_pages_and_slots_used_again(setups, name, dtype):
    """Up to three live requests in three slots and a pool just large enough: portions beside decoded tokens, requests
    left out of steps, pages handed to the next request without being cleared (unowned pages hold NaN)."""
    folder, requests, logits, upto = setups(name, dtype)
    many = dict(requests)
    many.update({rid + "again": ids for rid, ids in requests.items()})            # the same requests once more, in other slots
    plain_logits = dict(logits)
    plain_logits.update({rid + "again": logits[rid] for rid in requests})
    for seed in (3, 4):
        steps, where, peak = helpers.trace_mixed(many, seed, max_live=3, tail=10, page_tokens=16)
        ex = executor(folder, dtype, peak // 16, 16, max_requests=3, max_tokens=272)
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
    """Two tokens, then 300 one by one over pages of 16: the blocks and windows from the very first tokens, the rotations
    far from the start, pages the masks have left behind."""
    from bare_cuda_4gib_amd.engine import StepEntry
    folder, _, _, _ = setups(name, dtype)
    model = plain.PlainLagusun(folder)
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
    if name == "A":          # (the blocks and windows have left all but the last pages)
        assert ex.cache.pages_in_use(("block", 33)) <= 3 and ex.cache.pages_in_use(("window", 20)) <= 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point_and_the_scheduler(setups, dtype):
    from bare_cuda_4gib_amd.engine import Engine, generate_batch
    folder, _, _, _ = setups("A", dtype)
    model = plain.PlainLagusun(folder)
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
    """bin/llm-infer over a Lagusun folder: the architecture is chosen by config.json, ids in, ids out."""
    import os
    import subprocess
    import sys
    folder, _, _, _ = setups("B", "float32")
    model = plain.PlainLagusun(folder)
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
    got = helpers.replay_subprocess(folder, "float32", steps, str(tmp_path / "out"), peak, lagusun_models.CONFIGS["A"]["vocab"])
    close_rows(got, where, logits, "float32", "bin/trace_run", upto=upto)


# ---- the kernels of each mechanism alone ---------------------------------------------------------------------------

def step_context(lengths, cached, slots):
    """What the kernels read of a step's context: request s brings lengths[s] rows after cached[s] tokens, in slot slots[s]."""
    starts = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    row_seq = np.concatenate([np.full(n, s, dtype=np.int32) for s, n in enumerate(lengths)])
    positions = np.concatenate([np.arange(c, c + n, dtype=np.int32) for c, n in zip(cached, lengths)])
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=DEV)      # noqa: E731
    return types.SimpleNamespace(
        n_tokens=int(starts[-1]), n_seqs=len(lengths), row_seq=i32(row_seq), positions=i32(positions), token_ids=None,
        seq_start=list(starts), seq_ctx=list(cached), seq_slots=list(slots), seq_start_dev=i32(starts), seq_slots_dev=i32(slots),
        seq_ctx_dev=i32(cached), max_kv_len=int(max(c + n for c, n in zip(cached, lengths))), captured=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("channels,groups", [(36, 3), (37, 1), (64, 4), (2500, 5), (4096, 2), (24, 24)])
def test_norm_in_groups(dtype, channels, groups):
    """Every run of a row brought to unit mean square by itself -- one run made a hundred times larger than the others
    leaves them as they are --, on all rows and on chosen ones."""
    from bare_cuda_4gib_amd.engine.spec import PartSpec
    from bare_cuda_4gib_amd.parts import build_part
    torch.manual_seed(channels)
    x, g = torch.randn(9, channels) * 3.0, (torch.randn(channels) * 0.3 + 1.0).to(dtype)
    x[:, :channels // groups] *= 100.0
    part = build_part("norm", PartSpec("rmsnorm", dict(size=channels, eps=1e-3, groups=groups)))
    part.bind({"weight": g.to(DEV)}, types.SimpleNamespace(act_dtype=dtype, device=DEV))
    want = plain.grouped_norm(x.double(), g.double(), 1e-3, groups)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert torch.allclose(part.forward(x.to(DEV)).float().cpu().double(), want, atol=tol, rtol=tol)
    rows = torch.tensor([7, 0, 3, 3], dtype=torch.int32, device=DEV)
    assert torch.allclose(part.forward(x.to(DEV), rows=rows, n_rows=3).float().cpu().double(), want[[7, 0, 3]], atol=tol, rtol=tol)
    if groups > 1:
        assert float((want - plain.grouped_norm(x.double(), g.double(), 1e-3, 1)).abs().max()) > 0.5
        assert part.fusable() is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("channels,groups", [(36, 3), (37, 1), (64, 4), (4100, 1), (8192, 2), (2500, 5)])
@pytest.mark.parametrize("how", ["scaled", "plain", "replaced"])
def test_the_stream_s_update_and_the_norm_behind_it_in_one_kernel(dtype, channels, groups, how):
    """x += a * y (a sublayer's scaled output), x += y, and x = y + b (the stream replaced before a pass), each alone and
    with the next reader's norm in groups computed on the way."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(channels + groups)
    x, y = torch.randn(7, channels) * 2.0, torch.randn(7, channels)
    a, b, g = torch.randn(channels) * 0.5 + 1.0, torch.randn(channels), (torch.randn(channels) * 0.3 + 1.0).to(dtype)
    kw = dict(scaled=dict(scale=a.to(DEV)), plain={}, replaced=dict(bias=b.to(DEV), keep=False))[how]
    new = dict(scaled=x.double() + a.double() * y.double(), plain=(x + y).double(), replaced=y.double() + b.double())[how]
    want = plain.grouped_norm(new, g.double(), 1e-4, groups)
    xs = x.clone().to(DEV)
    assert ops.stream_update(xs, y.to(DEV), **kw) is None
    assert torch.allclose(xs.cpu().double(), new, atol=1e-6, rtol=1e-6)
    xs = x.clone().to(DEV)
    got = ops.stream_update(xs, y.to(DEV), norm_weight=g.to(DEV), eps=1e-4, groups=groups, out_dtype=dtype, **kw)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert torch.allclose(xs.cpu().double(), new, atol=1e-6, rtol=1e-6)
    assert got.dtype == dtype and torch.allclose(got.float().cpu().double(), want, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_embedding_s_factor_and_the_stream_replaced_before_a_pass(dtype):
    from bare_cuda_4gib_amd.engine.spec import PartSpec
    from bare_cuda_4gib_amd.parts import build_part
    torch.manual_seed(3)
    V, W, T, factor = 30, 40, 11, 3.25
    rt = types.SimpleNamespace(act_dtype=dtype, device=torch.device(DEV), place_weight=lambda t: t.to(DEV))
    table = torch.randn(V, W).to(dtype)
    emb = build_part("embedding", PartSpec("embedding", dict(vocab_size=V, hidden_size=W, scale=factor)))
    emb.bind({"weight": table.to(DEV)}, rt)
    ids = torch.randint(0, V, (T,), dtype=torch.int32)
    ctx = types.SimpleNamespace(token_ids=ids.to(DEV))
    x0 = table.double()[ids.long()] * factor
    assert torch.allclose(emb.forward(ctx).cpu().double(), x0, atol=1e-6, rtol=1e-6)
    re = build_part("reentry", PartSpec("stream_reentry", dict(hidden_size=W, passes=3)))
    w_in, steps = (torch.randn(W, 2 * W) / math.sqrt(2 * W)).to(dtype), torch.randn(3, W).to(dtype)
    re.bind({"in": w_in.to(DEV), "step": steps.to(DEV)}, rt)
    norm = build_part("norm", PartSpec("rmsnorm", dict(size=W, eps=1e-5, groups=4)))
    g = (torch.randn(W) * 0.2 + 1.0).to(dtype)
    norm.bind({"weight": g.to(DEV)}, rt)
    x = torch.randn(T, W) * 2.0
    rounded = lambda t: t.to(dtype).double()      # noqa: E731  (the product's operands are in the activations' dtype)
    want = torch.cat([rounded(x), rounded(x0.float())], dim=1) @ w_in.double().T + steps.double()[2]
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    xs = x.clone().to(DEV)
    assert re.forward(xs, ctx, emb, 2) is None
    assert torch.allclose(xs.cpu().double(), want, atol=tol, rtol=tol)
    xs = x.clone().to(DEV)
    made = re.forward(xs, ctx, emb, 2, norm)
    assert torch.allclose(xs.cpu().double(), want, atol=tol, rtol=tol)
    assert torch.allclose(made.float().cpu().double(), plain.grouped_norm(xs.cpu().double(), g.double(), 1e-5, 4), atol=tol, rtol=tol)
    assert float((want - (torch.cat([rounded(x), rounded(x0.float())], dim=1) @ w_in.double().T + steps.double()[0])).abs().max()) > 0.5


def rotary_table(positions, dims, base, scaling):
    from bare_cuda_4gib_amd.engine.spec import PartSpec
    from bare_cuda_4gib_amd.parts import build_part
    part = build_part("position", PartSpec("rotary", dict(theta=base, dim=dims, scaling=scaling)))
    return part.table(types.SimpleNamespace(positions=positions.to(DEV), shared=lambda key, make: make()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,dims,base,scaling", [(3, 8, 8, 10000.0, None), (2, 48, 24, 500.0, (6.0, 1.0, 3.0, 64)),
                                                         (5, 7, 6, 30.0, (2.0, 0.5, 2.0, 16)), (1, 130, 2, 7.0, None), (4, 10, 0, 1.0, None)])
def test_queries_and_keys_normed_over_the_whole_projection_then_rotated(dtype, heads, dim, dims, base, scaling):
    """The norm runs over all heads at once with a weight that spans them (one head made large shrinks the others), then
    the halves of the rotated part turn; into a dense tensor and into scattered cache slots, at position 70,001 too."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(dim)
    T, P, eps = 6, 4, 1e-2
    wide = (torch.randn(T, heads * dim + 11) * 0.2).to(dtype)
    wide[:, 5:5 + dim] *= 10.0
    x = wide[:, 5:5 + heads * dim]
    w = torch.randn(heads * dim) * 0.3 + 1.0
    positions = torch.tensor([0, 1, 2, 1000, 70001, 3], dtype=torch.int32)
    as_dict = dict(zip(("factor", "low", "high", "original"), scaling)) if scaling else None
    table = rotary_table(positions, dims, base, as_dict) if dims else None
    freqs = plain.scaled_frequencies(dims, base, as_dict)
    normed = (plain.unit_rms(x.double(), eps) * w.double()).view(T, heads, dim)
    want = plain.half_rotation(normed, positions, freqs)
    out = torch.zeros(T, heads, dim, device=DEV)
    ops.heads_prepare(wide.to(DEV)[:, 5:5 + heads * dim], heads, dim, out, norm_weight=w.to(DEV), norm_rows=True, table=table, eps=eps)
    assert torch.allclose(out.cpu().double(), want, atol=3e-5, rtol=3e-5)
    if heads > 1:      # (a norm a head would not pass)
        assert float((plain.half_rotation(plain.unit_rms(x.double().view(T, heads, dim), eps) * w.double().view(heads, dim), positions, freqs)
                      - want).abs().max()) > 0.1
    slot_map = torch.tensor([9, 2, 0, 7, 5, 11], dtype=torch.int32)
    cache = torch.zeros(3, heads, P, dim, dtype=dtype, device=DEV)
    ops.heads_prepare(wide.to(DEV)[:, 5:5 + heads * dim], heads, dim, cache, norm_weight=w.to(DEV), norm_rows=True, table=table,
                      slot_map=slot_map.to(DEV), page_tokens=P, eps=eps)
    tol = 3e-5 if dtype == torch.float32 else 1e-2
    flat = cache.cpu().double().permute(0, 2, 1, 3).reshape(3 * P, heads, dim)
    for t in range(T):
        assert torch.allclose(flat[slot_map[t]], want[t], atol=tol, rtol=tol), t


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,dims", [(3, 8, 8), (2, 48, 24), (5, 7, 6), (1, 130, 2), (4, 10, 0)])
def test_a_bias_then_the_rotation_then_the_unit_norm_a_head(dtype, heads, dim, dims):
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(dim + 1)
    T, eps = 5, 1e-2
    x, b = (torch.randn(T, heads * dim) * 0.2).to(dtype), torch.randn(heads * dim) * 0.2
    positions = torch.tensor([0, 1, 33, 1000, 70001], dtype=torch.int32)
    scaling = dict(factor=5.0, low=1.0, high=3.0, original=64)
    table = rotary_table(positions, dims, 50.0, scaling) if dims else None
    freqs = plain.scaled_frequencies(dims, 50.0, scaling)
    want = plain.unit_rms(plain.half_rotation((x.double() + b.double()).view(T, heads, dim), positions, freqs), eps)
    out = torch.zeros(T, heads, dim, device=DEV)
    ops.heads_prepare(x.to(DEV), heads, dim, out, bias=b.to(DEV), table=table, unit_after=True, eps=eps)
    assert torch.allclose(out.cpu().double(), want, atol=3e-5, rtol=3e-5)
    values = torch.zeros(T, heads, dim, device=DEV)                      # the values: a bias and the unit norm, nothing turned
    ops.heads_prepare(x.to(DEV), heads, dim, values, bias=b.to(DEV), unit_after=True, eps=eps)
    assert torch.allclose(values.cpu().double(), plain.unit_rms((x.double() + b.double()).view(T, heads, dim), eps), atol=3e-5, rtol=3e-5)


def paged(rows_k, rows_v, pages, P, dtype, n_pages):
    """Caches [pages, heads, P, size] that hold NaN but for the given rows, laid into the given pages."""
    k = torch.full((n_pages, rows_k.shape[1], P, rows_k.shape[2]), float("nan"), dtype=dtype, device=DEV)
    v = torch.full((n_pages, rows_v.shape[1], P, rows_v.shape[2]), float("nan"), dtype=dtype, device=DEV)
    for j in range(rows_k.shape[0]):
        if pages[j // P] >= 0:
            k[pages[j // P], :, j % P] = rows_k[j].to(dtype).to(DEV)
            v[pages[j // P], :, j % P] = rows_v[j].to(dtype).to(DEV)
    return k, v


def plain_row(kind, q, keys, values, pos, G, scale, size, cap=0.0, point=None):
    """The plain result for the row at position ``pos`` (the last of pos + 1 tokens): q [H, d], keys [n, G, d], values
    [n, G, e] -> ([H * e], weights [H, pos + 1]).  ``kind`` "block": softmax with a one in the denominator over the row's
    block of ``size`` positions; "window": sigmoid(capped score + point) over the last ``size`` keys.  size 0: every key."""
    H, n = q.shape[0], pos + 1
    qs = torch.zeros(n, H, q.shape[1], dtype=torch.float64)
    qs[-1] = q.double()
    s = plain.scores_of(qs, keys[:n].double(), H, G, scale)
    if kind == "block":
        w = plain.softmax_plus_one(s, plain.block_mask(n, size if size else n))
    else:
        if cap:
            s = plain.capped(s, cap)
        w = plain.sigmoid_weights(s, plain.window_mask(n, size if size else n), point.double())
    return plain.per_head(w, values[:n].double(), H, G)[-1], w[:, -1, :]


def run_rows(kind, q_rows, k_cache, v_cache, table, ctx, H, G, d, e, scale, size, cap=0.0, point=None, waves=0):
    from bare_cuda_4gib_amd.csrc import ops
    t = q_rows.shape[0]
    q = q_rows.view(t, H, 1, d).contiguous().float().to(DEV)
    if kind == "block":
        return ops.attention_maps(q, k_cache, v_cache, table, ctx, torch.float32, H, G, 1, d, e, 0, 0, scale, block=size, waves=waves,
                                  sink=torch.zeros(H, device=DEV)).cpu().double()
    return ops.attention_maps(q, k_cache, v_cache, table, ctx, torch.float32, H, G, 1, d, e, size, 0, scale, cap=cap, waves=waves,
                              point=point.float().to(DEV)).cpu().double()


SIZES = [(4, 2, 12, 20), (3, 3, 10, 70), (6, 1, 44, 100), (2, 1, 7, 130), (2, 2, 72, 200), (12, 4, 6, 9)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["block", "window"])
@pytest.mark.parametrize("sizes", SIZES)
@pytest.mark.parametrize("needle", [0, 7, 8, 63, 64, 120, 199])
def test_attention_finds_one_key_among_hundreds(dtype, kind, needle, sizes):
    """200 cached keys in scattered pages of 8, nothing masked; one key, far back, at a page's border or the row's own, is
    made to score far above the others in one head: with the softmax that head's weight goes there, with the sigmoid
    weights that key weighs nearly one among keys that weigh little; every head equals the plain result.  As a decoded
    token and as the last rows of a portion, with one wave and with eight cutting the keys."""
    torch.manual_seed(needle)
    (H, G, d, e), n, P, scale = sizes, 200, 8, 0.3
    if kind == "block":
        e = d
    keys, values = (torch.randn(n, G, d) * 0.3).to(dtype).float(), torch.randn(n, G, e).to(dtype).float()
    q = torch.randn(H, d)
    point = torch.randn(H) - 4.0
    mark = min(1, H - 1)
    keys[needle, mark // (H // G)] = (q[mark] / float(q[mark] @ q[mark]) * 20.0 / scale).to(dtype).float()
    pages = torch.randperm(40)[:n // P]
    k_cache, v_cache = paged(keys, values, pages, P, dtype, 40)
    table = pages.to(torch.int32).view(1, -1).to(DEV)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for lengths, cached, waves in (([1], [n - 1], 0), ([6], [n - 6], 1), ([2], [n - 2], 8)):
        ctx = step_context(lengths, cached, [0])
        got = run_rows(kind, q.view(1, H, d).repeat(lengths[0], 1, 1), k_cache, v_cache, table, ctx, H, G, d, e, scale, 0, 0.0, point, waves)
        for r in range(lengths[0]):
            pos = cached[0] + r
            want, weights = plain_row(kind, q, keys, values, pos, G, scale, 0, 0.0, point)
            assert torch.allclose(got[r], want, atol=tol * max(1.0, float(want.abs().max())), rtol=tol), (needle, pos)
            if needle <= pos:
                assert float(weights[mark][needle]) > 0.9


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("size", [1, 2, 6, 16, 50, 63, 64, 65, 100, 149])
@pytest.mark.parametrize("where", ["inside", "outside"])
def test_attention_at_the_edges_of_the_block(dtype, size, where):
    """The first key of the row's block, made to stand out, takes the weight; the key before it -- the last of the block
    before -- is not seen at all, and the one in the denominator takes what the few keys in sight leave.  Blocks count from
    position 0 whatever the step's rows: as a decoded token, and in a portion that crosses a block's border (every row
    with its own block), over scattered pages of 16, some of them given back (they hold NaN)."""
    torch.manual_seed(size)
    H, G, d, n, P, scale = 4, 2, 12, 150, 16, 0.3
    keys, values = (torch.randn(n, G, d) * 0.3).to(dtype).float(), torch.randn(n, G, d).to(dtype).float()
    q = torch.randn(H, d)
    pos_last = n - 1
    start = pos_last - pos_last % size
    needle = start if where == "inside" else start - 1
    if needle >= 0:
        keys[needle, 0] = (q[0] / float(q[0] @ q[0]) * 20.0 / scale).to(dtype).float()        # (head 0 reads key/value head 0)
    pages = torch.randperm(20)[:-(-n // P)]
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for lengths, cached in (([1], [n - 1]), ([5], [n - 5])):
        live = pages.clone()
        first_read = (cached[0] - cached[0] % size) // P          # pages before the first row's block went back
        live[:first_read] = -1
        k_cache, v_cache = paged(keys, values, live, P, dtype, 20)
        ctx = step_context(lengths, cached, [0])
        got = run_rows("block", q.view(1, H, d).repeat(lengths[0], 1, 1), k_cache, v_cache, live.to(torch.int32).view(1, -1).to(DEV), ctx,
                       H, G, d, d, scale, size)
        for r in range(lengths[0]):
            pos = cached[0] + r
            want, weights = plain_row("block", q, keys, values, pos, G, scale, size)
            assert torch.allclose(got[r], want, atol=tol * max(1.0, float(want.abs().max())), rtol=tol), (where, pos)
            assert float(weights[1].sum()) < 1.0 and int((weights[1] > 0).sum()) == pos % size + 1
            if pos == pos_last and needle >= 0:
                if where == "inside":
                    assert float(weights[0][needle]) > 0.9
                else:
                    assert float(weights[0][needle]) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 6, 9, 50, 63, 64, 65, 96, 130])
@pytest.mark.parametrize("where", ["inside", "outside"])
@pytest.mark.parametrize("cap", [0.0, 2.5])
def test_sigmoid_weights_at_the_edges_of_the_window(dtype, window, where, cap):
    """A key made to stand out just inside the window weighs nearly one (with a cap: what the cap leaves of it); one
    place further back it is not seen at all.  Nothing is normalised: every other key keeps its own small weight."""
    torch.manual_seed(window)
    H, G, d, e, n, P, scale = 4, 2, 12, 20, 150, 16, 0.3
    keys, values = (torch.randn(n, G, d) * 0.3).to(dtype).float(), torch.randn(n, G, e).to(dtype).float()
    q = torch.randn(H, d)
    point = torch.randn(H) - 1.0
    pos_last = n - 1
    needle = pos_last - window + 1 if where == "inside" else pos_last - window
    keys[needle, 0] = (q[0] / float(q[0] @ q[0]) * 20.0 / scale).to(dtype).float()
    pages = torch.randperm(20)[:-(-n // P)]
    k_cache, v_cache = paged(keys, values, pages, P, dtype, 20)
    table = pages.to(torch.int32).view(1, -1).to(DEV)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for lengths, cached in (([1], [n - 1]), ([5], [n - 5])):
        ctx = step_context(lengths, cached, [0])
        got = run_rows("window", q.view(1, H, d).repeat(lengths[0], 1, 1), k_cache, v_cache, table, ctx, H, G, d, e, scale, window, cap, point)
        for r in range(lengths[0]):
            pos = cached[0] + r
            want, weights = plain_row("window", q, keys, values, pos, G, scale, window, cap, point)
            assert torch.allclose(got[r], want, atol=tol * max(1.0, float(want.abs().max())), rtol=tol), (where, pos)
            if pos == pos_last:
                if where == "inside":
                    top = 1.0 / (1.0 + math.exp(-(cap + float(point[0])))) if cap else 1.0
                    assert abs(float(weights[0][needle]) - top) < 1e-3
                else:
                    assert float(weights[0][needle]) == 0.0
                assert int((weights[1] > 0).sum()) == min(window, pos + 1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["block", "window"])
def test_attention_of_the_first_tokens_and_unequal_requests(dtype, kind):
    """Three requests in one step -- the first token of a sequence, a portion from position 0, a decoded token far in --
    each with a block table of its own.  The first token alone: with the softmax the one in the denominator halves...
    not quite -- it takes 1 / (1 + exp(s)) of the weight; with the sigmoid weights the token weighs sigmoid(s + b)."""
    torch.manual_seed(8)
    H, G, d, P, scale, size = 3, 3, 10, 4, 0.5, 5
    e = d if kind == "block" else 6
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
    point = torch.tensor([3.0, -3.0, 0.3])
    got = run_rows(kind, q, k_cache, v_cache, tables.to(DEV), ctx, H, G, d, e, scale, size, 0.0, point)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    row = 0
    for s, (new, old) in enumerate(zip(lengths, cached)):
        for i in range(new):
            want, weights = plain_row(kind, q[row], seqs[s][0], seqs[s][1], old + i, G, scale, size, 0.0, point)
            assert torch.allclose(got[row], want, atol=tol, rtol=tol), (s, i)
            if s == 0:
                sc = float(q[0, 0].double() @ seqs[0][0][0, 0].double()) * scale
                first = math.exp(sc) / (1.0 + math.exp(sc)) if kind == "block" else 1.0 / (1.0 + math.exp(-(sc + 3.0)))
                assert abs(float(weights[0][0]) - first) < 1e-9
            row += 1


@pytest.mark.parametrize("experts,top,factor", [(8, 3, 1.0), (6, 2, 2.5), (5, 5, 0.5), (4, 1, 1.0), (3, 2, 3.0), (64, 6, 1.5), (1, 1, 2.0), (40, 7, 1.0)])
def test_the_sigmoid_router_chooses_by_corrected_scores_and_weighs_by_the_plain_ones(experts, top, factor):
    """Logits of many rows with corrections large enough to change the choice; the weights are the chosen experts' plain
    scores over their sum, times the factor; rows whose choice is a close call in 32-bit are left out.  The logits are a
    part of wider rows."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(experts * 10 + top)
    T = 300
    wide = torch.randn(T, experts + 3) * 2.0
    correction = torch.randn(experts) * 0.3
    z = wide[:, :experts]
    chosen, weights, margin = plain.route(z.double(), correction.double(), top, factor)
    got_w, got_c = ops.moe_route(wide.to(DEV)[:, :experts], experts, top, 1, 1, correction.to(DEV), want_chosen=True, squash=True,
                                 normalize=True, factor=factor)
    got_w, got_c = got_w.cpu().double(), got_c.cpu().long()
    want_w = torch.zeros(T, experts, dtype=torch.float64).scatter_(1, chosen, weights)
    sure = margin > 1e-5
    assert int(sure.sum()) > T * 0.9
    assert torch.allclose(got_w[sure], want_w[sure], atol=1e-6, rtol=1e-5)
    assert torch.equal(got_c[sure].sort(dim=1).values, chosen[sure].sort(dim=1).values)
    assert bool(((got_w > 0).sum(dim=1) == top).all())
    assert torch.allclose(got_w.sum(dim=1), torch.full((T,), factor, dtype=torch.float64), atol=1e-5)
    if 1 < top < experts:         # (the correction matters, and so does the sigmoid: a softmax's weights would differ)
        plain_choice, _, _ = plain.route(z.double(), torch.zeros(experts, dtype=torch.float64), top, factor)
        assert not torch.equal(plain_choice.sort(dim=1).values, chosen.sort(dim=1).values)
        soft = torch.softmax(z.double(), -1).gather(1, chosen)
        assert float((soft / soft.sum(-1, keepdim=True) * factor - weights).abs().max()) > 1e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,ff,shared_ff", [(3, 10, 7), (4, 16, 0), (1, 5, 3), (6, 24, 16), (0, 0, 12)])
def test_weighted_gelu_units_and_the_shared_one(dtype, experts, ff, shared_ff):
    """Every expert's units times the row's weight for it (zero where it was not chosen), the shared unit's as they are;
    the exact gelu, not the tanh form; in place too."""
    from bare_cuda_4gib_amd.csrc import ops
    torch.manual_seed(experts + ff)
    T = 13
    z = (torch.randn(T, experts * ff + shared_ff) * 2.0).to(dtype)
    weights = torch.rand(T, experts) * (torch.rand(T, experts) > 0.4) if experts else None
    want = []
    for j in range(experts):
        want.append(plain.exact_gelu(z[:, ff * j:ff * (j + 1)].double()) * weights[:, j:j + 1].double())
    if shared_ff:
        want.append(plain.exact_gelu(z[:, ff * experts:].double()))
    want = torch.cat(want, dim=1)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    zd = z.to(DEV)
    got = ops.routed_gelu(zd, weights.float().to(DEV) if experts else None, experts, ff, shared_ff).float().cpu().double()
    assert got.shape == want.shape and torch.allclose(got, want, atol=tol, rtol=tol)
    assert ops.routed_gelu(zd, weights.float().to(DEV) if experts else None, experts, ff, shared_ff, out=zd) is zd
    assert torch.allclose(zd.float().cpu().double(), want, atol=tol, rtol=tol)
    if dtype == torch.float32 and shared_ff:
        zz = z[:, ff * experts:].double()
        tanh_form = 0.5 * zz * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (zz + 0.044715 * zz ** 3)))
        assert float((got[:, ff * experts:] - tanh_form).abs().max()) > 1e-4
