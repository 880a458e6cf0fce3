"""Napadra through the framework against the plain implementation of tests/plain/napadra_plain.py.

Every test runs on three backends: the engine on the CPU with the plain torch ops standing in for the kernel
library (the host side: tables, slots, state, batching), and the engine on the GPU in float32 and in bfloat16 (the
HIP kernels).  The models are the tiny ones of napadra_configs.py with sharpened weights.
"""
import numpy as np
import pytest
import torch

import trace_tools as tt
from napadra_configs import NAPADRA, write_model
from plain import napadra_plain as plain
from tiny_configs import random_ids

BACKENDS = [pytest.param("cpu", id="cpu"),
            pytest.param("gpu-float32", marks=pytest.mark.gpu, id="gpu-float32"),
            pytest.param("gpu-bfloat16", marks=pytest.mark.gpu, id="gpu-bfloat16")]
# Against logits of order 1: float32 sums in another order.  bfloat16 rounds the activations between the kernels, and the
# sharpened weights carry that further than a trained model's would: there the bound is on each row's root mean square
# error against the row's own spread (a key too many or a lost state moves a row by its whole spread; float32 pins
# the same kernels' indexing to five digits).
TOL = {"cpu": 2e-5, "gpu-float32": 5e-5, "gpu-bfloat16": 0.12}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("napadra")
    return {name: write_model(raw, seed, str(root / name)) for name, (raw, seed) in NAPADRA.items()}


@pytest.fixture(scope="module")
def oracle(folders):
    cache = {}

    def get(name, ids):
        key = (name, tuple(ids))
        if key not in cache:
            cfg, tensors = plain.load_folder(folders[name])
            cache[key] = plain.forward(cfg, tensors, list(ids)).to(torch.float32)
        return cache[key]
    return get


def make_engine(folder, backend, **kw):
    from tokenizer_amd.engine import Engine, load_model
    if backend == "cpu":
        from kernel_refs import PlainOps
        return Engine(load_model(folder, "float32", "cpu", ops=PlainOps()), **kw)
    return Engine(load_model(folder, backend.split("-")[1]), **kw)


def close(got, want, backend, what=""):
    got = got.float().cpu()
    if backend == "gpu-bfloat16":
        spread = (want - want.mean(dim=-1, keepdim=True)).pow(2).mean(dim=-1).sqrt()
        off = (got - want).pow(2).mean(dim=-1).sqrt() / spread
        # (A row here and there sits on an edge, a clamp or a maximum that two terms nearly share, where rounding
        # tips it; the same rows are off by as much however the prompt is cut.  Such rows are few.)
        assert float(off.max()) <= 4 * TOL[backend] and int((off > TOL[backend]).sum()) <= max(1, off.numel() // 50), \
            f"{what}: rows are off by up to {float(off.max())} of their spread, {int((off > TOL[backend]).sum())} over the bound"
        return
    err = float((got - want).abs().max())
    bound = TOL[backend] * max(float(want.abs().max()), 1.0)
    assert err <= bound, f"{what}: max abs error {err} against a bound of {bound}"


def requests_for(name, lengths=(1, 2, 3, 21, 50, 97, 64, 33)):
    vocab = NAPADRA[name][0]["vocab"]
    return {f"r{i}": random_ids(vocab, n, 40 + i) for i, n in enumerate(lengths)}


def check_trace(folders, oracle, name, backend, steps, reqs, **kw):
    eng = make_engine(folders[name], backend, max_tokens=tt.peak_tokens(steps), max_requests=4, **kw)
    eng.pools.poison()          # pages and state rows that no request wrote read as NaN
    got = tt.run_in_process(eng, steps)
    for rid, ids in reqs.items():
        close(got[rid], oracle(name, ids), backend, rid)
    eng.cache.check_invariants()
    assert not eng.cache.requests
    return eng


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", list(NAPADRA))
def test_whole_prompts_and_the_first_tokens(folders, oracle, name, backend):
    reqs = requests_for(name)
    check_trace(folders, oracle, name, backend, tt.whole(reqs), reqs)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", list(NAPADRA))
def test_prefill_then_token_by_token(folders, oracle, name, backend):
    # The tail of 40 passes every chunk edge of the models (5, 7, 20, 33, 48) and page borders of 16.
    reqs = requests_for(name, (50, 97, 64, 41))
    check_trace(folders, oracle, name, backend, tt.decode_tail(reqs, 40), reqs)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", list(NAPADRA))
@pytest.mark.parametrize("seed", [3, 4])
def test_portions_down_to_two_tokens(folders, oracle, name, backend, seed):
    reqs = requests_for(name, (97, 50, 64, 7))
    steps = tt.portions(reqs, seed)
    assert any(len(s["entries"][0]["tokens"]) == 2 for s in steps)
    check_trace(folders, oracle, name, backend, steps, reqs)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", list(NAPADRA))
@pytest.mark.parametrize("seed", [6, 7])
def test_mixed_batches_with_pages_and_slots_used_again(folders, oracle, name, backend, seed):
    reqs = requests_for(name, (33, 97, 21, 64, 50, 80, 12, 45, 3, 70))
    steps = tt.mixed(reqs, seed, max_live=4, tail=14)
    assert max(len(s["entries"]) for s in steps) >= 3
    eng = check_trace(folders, oracle, name, backend, steps, reqs)
    assert eng.cache.max_requests == 4          # ten requests went through four slots


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("page_size", [16, 48])
def test_other_page_sizes_and_batches_against_each_request_alone(folders, oracle, backend, page_size):
    from tokenizer_amd.engine import StepEntry
    name = "R"
    reqs = requests_for(name, (70, 9, 31))
    eng = make_engine(folders[name], backend, num_pages=24, page_size=page_size, max_requests=3)
    eng.pools.poison()
    for rid in reqs:
        eng.add_request(rid)
    heads = {rid: len(ids) - 5 for rid, ids in reqs.items()}
    got = {rid: [] for rid in reqs}
    logits = eng.step([StepEntry(rid, ids[:heads[rid]], list(range(heads[rid]))) for rid, ids in reqs.items()]).float().cpu()
    row = 0
    for rid in reqs:
        got[rid].append(logits[row:row + heads[rid]])
        row += heads[rid]
    for k in range(5):
        logits = eng.step([StepEntry(rid, [ids[heads[rid] + k]], [0]) for rid, ids in reqs.items()]).float().cpu()
        for row, rid in enumerate(reqs):
            got[rid].append(logits[row:row + 1])
    for rid, ids in reqs.items():
        close(torch.cat(got[rid]), oracle(name, ids), backend, rid)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["P", "Q"])
def test_long_decoding(folders, oracle, name, backend):
    ids = random_ids(NAPADRA[name][0]["vocab"], 230, 77)
    reqs = {"long": ids}
    check_trace(folders, oracle, name, backend, tt.decode_tail(reqs, tail=227), reqs)


@pytest.mark.parametrize("backend", BACKENDS)
def test_greedy_generation_through_the_entry_point_and_the_scheduler(folders, backend):
    from tokenizer_amd.engine import GenerateParams, Scheduler, SchedulerConfig, generate
    name = "P"
    cfg, tensors = plain.load_folder(folders[name])
    prompts = [random_ids(cfg["vocab"], n, 90 + n) for n in (11, 30, 4)]
    want = [plain.greedy_generate(cfg, tensors, p, 9) for p in prompts]
    eng = make_engine(folders[name], backend, num_pages=16, max_requests=4)
    eng.pools.poison()
    alone = [generate(eng, p, GenerateParams.greedy(9)).tokens for p in prompts]
    sched = Scheduler(eng, SchedulerConfig(num_blocks=16, max_batch_size=4))
    rids = [sched.add_request(p, GenerateParams.greedy(9)) for p in prompts]
    results = sched.run()
    together = [results[rid].tokens for rid in rids]
    assert alone == together
    if backend != "gpu-bfloat16":           # (bfloat16 may pick another of two near-equal logits)
        assert alone == want
    else:
        assert sum(a == w for a, w in zip(sum(alone, []), sum(want, []))) >= 20


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_hundreds_of_tokens_with_long_chunks(folders, oracle, dtype, cut):
    """Contexts of up to 900 tokens under chunks of 300, 520 and 1,024: keys far back inside a chunk, chunk edges deep in a
    prompt and among decoded tokens, the decayed memory of hundreds of tokens."""
    name = "U"
    reqs = {f"r{i}": random_ids(NAPADRA[name][0]["vocab"], n, 70 + i) for i, n in enumerate((900, 333, 610, 545))}
    steps = {"whole": lambda: tt.whole(reqs), "tail": lambda: tt.decode_tail(reqs, 48),
             "portions": lambda: tt.portions(reqs, 9), "mixed": lambda: tt.mixed(reqs, 12, max_live=3, tail=30)}[cut]()
    check_trace(folders, oracle, name, "gpu-" + dtype, steps, reqs)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_replay_program_on_a_model_folder(folders, oracle, tmp_path, dtype):
    """bin/trace_run as a child process: the class is chosen by config.json, the pool is made for the trace's peak,
    four state slots serve ten requests."""
    name = "T"
    reqs = requests_for(name, (33, 97, 21, 64, 50, 80, 12, 45, 3, 70))
    steps = tt.mixed(reqs, 11, max_live=4, tail=14)
    got = tt.run_program(folders[name], dtype, steps, str(tmp_path / "out"), tt.peak_tokens(steps), NAPADRA[name][0]["vocab"])
    for rid, ids in reqs.items():
        close(got[rid], oracle(name, ids), "gpu-" + dtype, rid)


# ------------------------------------------------------------------ mechanisms alone
def ops_for(backend):
    if backend == "cpu":
        from kernel_refs import PlainOps
        return PlainOps(), torch.device("cpu"), torch.float32
    from tokenizer_amd.kernels import get_ops
    return get_ops(), torch.device("cuda:0"), (torch.float32 if backend.endswith("float32") else torch.bfloat16)


def rounded(x, dtype):
    """Random float64 data as the compute dtype holds it."""
    return x.to(dtype).to(torch.float64)


class Batch:
    """A batch description made by hand: entries of (first position, rows, slot)."""

    def __init__(self, entries, device):
        i32 = lambda values: torch.tensor(values, dtype=torch.int32, device=device)
        self.cu_q = i32(np.cumsum([0] + [n for _, n, _ in entries]).tolist())
        self.first_position = i32([p for p, _, _ in entries])
        self.state_slots = i32([s for _, _, s in entries])
        self.entry_of_token = i32([e for e, (_, n, _) in enumerate(entries) for _ in range(n)])
        self.positions = i32([p + k for p, n, _ in entries for k in range(n)])
        self.n_tokens = int(self.cu_q[-1])
        tiles = [[e, at] for e, (_, n, _) in enumerate(entries) if n != 1 for at in range(0, n, 16)]
        self.q_tiles = i32(tiles).reshape(-1, 2)
        rows = np.cumsum([0] + [n for _, n, _ in entries])
        self.decode_rows = i32([int(rows[e]) for e, (_, n, _) in enumerate(entries) if n == 1])
        self.max_position = max(p + n - 1 for p, n, _ in entries)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width,streams", [(64, 2), (200, 3), (4352, 1), (24, 8), (52, 13)])
def test_streams_step_alone(backend, width, streams):
    from tokenizer_amd.parts.streams import StreamWrite
    ops, device, dtype = ops_for(backend)
    gen = torch.Generator().manual_seed(width)
    rand = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float64)
    tokens = 5
    x = rand(tokens, streams, width).to(torch.float32).to(torch.float64)
    y, mix, out_c, read = rounded(rand(tokens, width), dtype), rand(streams, streams).float().double(), \
        rand(streams).float().double(), rand(streams).float().double()
    scale, gain, eps = rand(width).float().double(), torch.tensor([1.7], dtype=torch.float64), 1e-5
    new = torch.einsum("tsw,sr->trw", x, mix) + out_c[None, :, None] * (scale * y)[:, None, :]
    want = plain.scalar_norm(torch.einsum("tsw,s->tw", new, read), gain, eps)
    dev = lambda t, kind=torch.float32: t.to(kind).to(device)
    held = dev(x)
    got = torch.empty((tokens, width), dtype=dtype, device=device)
    ops.streams_step(held, StreamWrite(dev(y, dtype), dev(mix), dev(out_c), dev(scale)), dev(read), dev(gain), eps, got)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
    assert float((got.double().cpu() - want).abs().max()) <= tol * float(want.abs().max())
    assert float((held.double().cpu() - new).abs().max()) <= 1e-5 * float(new.abs().max())
    # A subset of rows, nothing stored, no write pending: the read of the streams as they are.
    rows = torch.tensor([3, 0], dtype=torch.int32, device=device)
    got = torch.empty((2, width), dtype=dtype, device=device)
    before = held.clone()
    ops.streams_step(held, None, dev(read), dev(gain), eps, got, rows=rows)
    want = plain.scalar_norm(torch.einsum("tsw,s->tw", new[[3, 0]], read), gain, eps)
    assert float((got.double().cpu() - want).abs().max()) <= tol * float(want.abs().max())
    assert torch.equal(before, held)


@pytest.mark.parametrize("backend", BACKENDS)
def test_token_shift_alone_with_state_across_steps(backend):
    ops, device, dtype = ops_for(backend)
    gen = torch.Generator().manual_seed(5)
    width, n = 40, 11
    h = torch.randn(2, n, width, generator=gen, dtype=torch.float64).float()
    mu = torch.rand(width, generator=gen, dtype=torch.float64).float()
    want = [plain.token_shift(h[r].double(), mu.double()) for r in range(2)]
    state = torch.full((3, width), float("nan"), device=device)
    # Request 0 in slot 2, request 1 in slot 0; cut 4 + 1 + 6 and 1 + 8 + 2; single rows go the fused way where there is one.
    cuts = {0: [4, 1, 6], 1: [1, 8, 2]}
    at, got = {0: 0, 1: 0}, {0: [], 1: []}
    for step in range(3):
        entries = [(at[r], cuts[r][step], slot) for r, slot in ((0, 2), (1, 0))]
        batch = Batch(entries, device)
        rows = torch.cat([h[r, at[r]:at[r] + cuts[r][step]] for r in (0, 1)]).to(device)
        out = torch.empty(rows.shape, dtype=dtype, device=device)
        ops.token_shift(rows, mu.to(device), state, batch.cu_q, batch.first_position, batch.state_slots,
                        batch.entry_of_token, out)
        row = 0
        for r in (0, 1):
            got[r].append(out[row:row + cuts[r][step]].double().cpu())
            row += cuts[r][step]
            at[r] += cuts[r][step]
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-6
    for r in (0, 1):
        assert float((torch.cat(got[r]) - want[r]).abs().max()) <= tol * 4


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,d,dv", [(2, 16, 24), (1, 40, 8), (3, 8, 72), (2, 256, 64)])
def test_matrix_memory_alone_in_portions(backend, heads, d, dv):
    ops, device, dtype = ops_for(backend)
    gen = torch.Generator().manual_seed(heads * d + dv)
    n, cap, eps, width = 37, 6.0, 1e-5, 32
    h = torch.randn(n, width, generator=gen, dtype=torch.float64)
    w = {name: torch.randn(rows, width, generator=gen, dtype=torch.float64) * 0.4
         for name, rows in (("q", heads * d), ("k", heads * d), ("v", heads * dv), ("g", heads * dv), ("i", heads), ("f", heads))}
    w["i.b"], w["f.b"] = torch.randn(heads, generator=gen, dtype=torch.float64), torch.randn(heads, generator=gen, dtype=torch.float64) + 2
    w["norm"] = torch.rand(heads * dv, generator=gen, dtype=torch.float64) + 0.5
    w["o"] = torch.eye(heads * dv, dtype=torch.float64)
    qkvg = rounded(torch.cat([h @ w[name].t() for name in "qkvg"], dim=1), dtype)
    gates = torch.cat([h @ w["i"].t() + w["i.b"], h @ w["f"].t() + w["f.b"]], dim=1).float().double()
    # The plain function makes its own projections: hand it weights that give back these rounded rows.
    pinv = torch.linalg.pinv(h)
    exact = dict(w)
    sizes = [heads * d, heads * d, heads * dv, heads * dv]
    for name, part in zip("qkvg", torch.split(qkvg, sizes, dim=1)):
        exact[name] = (pinv @ part).t()
    exact["i"], exact["f"] = (pinv @ (gates[:, :heads] - w["i.b"])).t(), (pinv @ (gates[:, heads:] - w["f.b"])).t()
    want = plain.mlstm(h, {"heads": heads, "dim": d, "vdim": dv, "gate_cap": cap}, exact, eps)
    state = torch.full((2, heads * d * dv + heads * d + heads + 3), float("nan"), device=device)
    got = []
    at = 0
    for size in (5, 1, 1, 17, 2, 11):
        batch = Batch([(at, size, 1)], device)
        rows = qkvg[at:at + size].to(dtype).to(device).contiguous()
        read = torch.empty((size, heads * dv), dtype=torch.float32, device=device)
        ops.mlstm_scan(rows, gates[at:at + size].float().to(device).contiguous(), state, batch.cu_q, batch.first_position,
                       batch.state_slots, read, heads, d, dv, cap)
        out = torch.empty((size, heads * dv), dtype=dtype, device=device)
        ops.head_norm_gate(read, w["norm"].float().to(device), rows, 2 * heads * d + heads * dv, eps, heads, dv, out)
        got.append(out.double().cpu())
        at += size
    tol = 3e-2 if dtype == torch.bfloat16 else 2e-4
    assert float((torch.cat(got) - want).abs().max()) <= tol * max(1.0, float(want.abs().max()))


def _memory_rows(seed, n, heads, d, dv, cap, eps, dtype, forget_shift=2.0):
    """Rows of q, k, v, g and gate pre-activations of one sequence as the compute dtype holds them, and what the plain
    function reads from them."""
    gen = torch.Generator().manual_seed(seed)
    sizes = [heads * d, heads * d, heads * dv, heads * dv]
    qkvg = rounded(torch.cat([torch.randn(n, size, generator=gen, dtype=torch.float64) * 0.8 for size in sizes], dim=1), dtype)
    gates = torch.randn(n, 2 * heads, generator=gen, dtype=torch.float64) * 3.0
    gates[:, heads:] += forget_shift
    gates = gates.float().double()
    w = {"norm": torch.rand(heads * dv, generator=torch.Generator().manual_seed(heads * dv), dtype=torch.float64) + 0.5, "o": torch.eye(heads * dv, dtype=torch.float64),
         "i.b": torch.zeros(heads, dtype=torch.float64), "f.b": torch.zeros(heads, dtype=torch.float64)}
    # The plain function makes its own projections: its input is the identity, its weights are the rows themselves.
    eye = torch.eye(n, dtype=torch.float64)
    for name, part in zip("qkvg", torch.split(qkvg, sizes, dim=1)):
        w[name] = part.t().contiguous()
    w["i"], w["f"] = gates[:, :heads].t().contiguous(), gates[:, heads:].t().contiguous()
    want = plain.mlstm(eye, {"heads": heads, "dim": d, "vdim": dv, "gate_cap": cap}, w, eps)
    return qkvg, gates, w["norm"], want


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,d,dv,shift", [(2, 16, 24, 2.0), (1, 72, 8, 4.0), (3, 12, 70, -1.0), (1, 130, 66, 6.0),
                                                (1, 300, 20, 3.0)])
def test_matrix_memory_in_long_portions_beside_single_tokens(backend, heads, d, dv, shift):
    """Two sequences whose portions run from one row to hundreds, side by side: long portions take the form in chunks of
    64 tokens, short ones the token-by-token form, and the state passes between the two from step to step."""
    ops, device, dtype = ops_for(backend)
    cap, eps = 7.0, 1e-5
    steps = [(130, 1), (70, 65), (1, 2), (99, 50), (64, 0), (1, 128), (3, 1)]
    lengths = [sum(a for a, _ in steps), sum(b for _, b in steps)]
    seqs = [_memory_rows(11 * heads + d + k, lengths[k], heads, d, dv, cap, eps, dtype, shift) for k in range(2)]
    state = torch.full((5, heads * d * dv + heads * d + heads + 1), float("nan"), device=device)
    slots, at, got = (3, 1), [0, 0], [[], []]
    for sizes in steps:
        live = [k for k in range(2) if sizes[k]]
        batch = Batch([(at[k], sizes[k], slots[k]) for k in live], device)
        rows = torch.cat([seqs[k][0][at[k]:at[k] + sizes[k]] for k in live]).to(dtype).to(device).contiguous()
        gate_rows = torch.cat([seqs[k][1][at[k]:at[k] + sizes[k]] for k in live]).float().to(device).contiguous()
        read = torch.empty((rows.shape[0], heads * dv), dtype=torch.float32, device=device)
        ops.mlstm_scan(rows, gate_rows, state, batch.cu_q, batch.first_position, batch.state_slots, read, heads, d, dv, cap)
        out = torch.empty((rows.shape[0], heads * dv), dtype=dtype, device=device)
        ops.head_norm_gate(read, seqs[0][2].float().to(device), rows, 2 * heads * d + heads * dv, eps, heads, dv, out)
        out = out.double().cpu()
        row = 0
        for k in live:
            got[k].append(out[row:row + sizes[k]])
            row += sizes[k]
            at[k] += sizes[k]
    tol = 3e-2 if dtype == torch.bfloat16 else 2e-4
    for k in range(2):
        want = seqs[k][3]
        assert float((torch.cat(got[k]) - want).abs().max()) <= tol * max(1.0, float(want.abs().max())), k


def _paged(ops, device, dtype, q, k, v, page_size, chunk, slopes, sinks, scale, first_page=3, as_prompt=False):
    """Attention of every row of q (positions 0..n-1 of one request) over keys and values laid into pages.
    `as_prompt`: the rows are described as one portion of a prompt (the kernels for portions then take them)."""
    n, n_q, d = q.shape
    n_kv, dv = k.shape[1], v.shape[2]
    n_pages = first_page + -(-n // page_size) + 1
    k_pages = torch.full((n_pages, n_kv, page_size, d), float("nan"), dtype=dtype, device=device)
    v_pages = torch.full((n_pages, n_kv, dv, page_size), float("nan"), dtype=dtype, device=device)
    table = list(range(n_pages - 1, first_page - 1, -1))[: -(-n // page_size)]      # pages in falling order
    for j in range(n):
        k_pages[table[j // page_size], :, j % page_size, :] = k[j].to(dtype).to(device)
        v_pages[table[j // page_size], :, :, j % page_size] = v[j].to(dtype).to(device)
    i32 = lambda values: torch.tensor(values, dtype=torch.int32, device=device)
    out = torch.empty((n, n_q * dv), dtype=dtype, device=device)
    f32 = lambda t: None if t is None else t.float().to(device)
    ops.paged_attention(q.reshape(n, -1).to(dtype).to(device).contiguous(), out, k_pages, v_pages, i32(list(range(n))),
                        i32([0] * n), i32([table]), n_q, n_kv, d, None, scale, max_position=n - 1,
                        batch=Batch([(0, n, 0)], device) if as_prompt else None,
                        value_dim=dv, chunk=chunk, slopes=f32(slopes), sinks=f32(sinks))
    return out.double().cpu().reshape(n, n_q, dv)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("as_prompt", [False, True])
@pytest.mark.parametrize("n_q,n_kv,d,dv,chunk,n", [(4, 2, 16, 24, 20, 75), (3, 3, 32, 32, 33, 75), (8, 1, 16, 8, 7, 75),
                                                   (2, 1, 80, 48, 300, 75), (4, 1, 64, 64, 21, 75), (34, 2, 128, 128, 50, 75),
                                                   (4, 2, 64, 64, 512, 700)])
def test_attention_alone_against_the_plain_function(backend, n_q, n_kv, d, dv, chunk, n, as_prompt):
    """(The last case is long enough for the single-token kernel to cut a token's keys over workgroups, with the sink in
    the first part's sums, and for several waves to share a tile's keys in the kernel for portions.)"""
    ops, device, dtype = ops_for(backend)
    if backend == "cpu" and n > 100:
        pytest.skip("the plain ops walk token by token: the long case is for the kernels")
    gen = torch.Generator().manual_seed(n_q + d)
    scale = 0.31
    h = torch.eye(n, dtype=torch.float64)                        # so that the projections' weights are q, k, v themselves
    q = rounded(torch.randn(n, n_q * d, generator=gen, dtype=torch.float64), dtype)
    k = rounded(torch.randn(n, n_kv * d, generator=gen, dtype=torch.float64), dtype)
    v = rounded(torch.randn(n, n_kv * dv, generator=gen, dtype=torch.float64), dtype)
    sinks = torch.randn(n_q, generator=gen, dtype=torch.float64).float().double() + 1.0
    mixer = {"heads": n_q, "kv_heads": n_kv, "dim": d, "vdim": dv, "scale": scale, "mask": {"size": chunk}}
    w = {"q": q.t(), "sink": sinks, "o": torch.eye(n_q * dv, dtype=torch.float64)}
    want = plain.attention(h, mixer, w, k.reshape(n, n_kv, d).transpose(0, 1), v.reshape(n, n_kv, dv).transpose(0, 1))
    got = _paged(ops, device, dtype, q.reshape(n, n_q, d), k.reshape(n, n_kv, d), v.reshape(n, n_kv, dv), 16, chunk,
                 plain.distance_slopes(n_q), sinks, scale, as_prompt=as_prompt)
    tol = 2e-2 if dtype == torch.bfloat16 else 2e-5
    assert float((got.reshape(n, -1) - want).abs().max()) <= tol * float(want.abs().max())


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dv,as_prompt", [(8, False), (16, False), (16, True)])
def test_one_key_that_stands_out_is_seen_just_inside_its_chunk_and_not_just_outside(backend, dv, as_prompt):
    """Every value is zero but one key's, whose score is made to stand far out: the output is that value (times what
    the sink and the bias leave) when the key lies in the query's chunk, and nothing when it lies just before it."""
    ops, device, dtype = ops_for(backend)
    n, chunk, d = 130, 48, 16
    for marked in (0, 47, 48, 63, 64, 95, 96, 127):             # chunk edges and page borders
        q = torch.zeros(n, 1, d, dtype=torch.float64)
        k = torch.zeros(n, 1, d, dtype=torch.float64)
        v = torch.zeros(n, 1, dv, dtype=torch.float64)
        q[:, 0, 0] = 8.0
        k[marked, 0, 0] = 8.0
        v[marked, 0, :] = 1.0
        got = _paged(ops, device, dtype, q, k, v, 16, chunk, torch.tensor([0.01]), torch.tensor([0.0]), 1.0,
                     as_prompt=as_prompt)[:, 0, 0]
        last_seen = (marked // chunk + 1) * chunk - 1
        for query in range(n):
            if marked <= query <= last_seen:
                assert got[query] > 0.99, (marked, query, float(got[query]))
            else:
                assert got[query] == 0.0, (marked, query, float(got[query]))


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_sink_takes_its_share_and_the_bias_grows_with_distance(backend):
    ops, device, dtype = ops_for(backend)
    n, d, dv = 20, 16, 16
    q, k = torch.zeros(n, 2, d, dtype=torch.float64), torch.zeros(n, 1, d, dtype=torch.float64)
    v = torch.ones(n, 1, dv, dtype=torch.float64)
    slopes, sinks = torch.tensor([0.5, 0.0]), torch.tensor([0.0, 2.0])
    got = _paged(ops, device, dtype, q, k, v, 16, None, slopes, sinks, 1.0)
    for query in range(n):
        # Head 0: keys at distance m weigh exp(-m / 2) beside a sink of weight 1; head 1: all keys 1 beside a sink of e^2.
        keys = sum(np.exp(-0.5 * m) for m in range(query + 1))
        assert abs(float(got[query, 0, 0]) - keys / (keys + 1.0)) < 1e-2
        assert abs(float(got[query, 1, 0]) - (query + 1) / (query + 1 + np.exp(2.0))) < 1e-2


@pytest.mark.parametrize("backend", BACKENDS)
def test_capped_gated_activation_and_position_vector_alone(backend):
    ops, device, dtype = ops_for(backend)
    gen = torch.Generator().manual_seed(9)
    for inner in (44, 72):            # rows of 72 are whole runs of sixteen bytes: the kernel that reads them so
        x = rounded(torch.randn(7, 2 * inner, generator=gen, dtype=torch.float64) * 2, dtype)
        out = torch.empty((7, inner), dtype=dtype, device=device)
        ops.silu_gate(x.to(dtype).to(device), out, act=(1.702, 0.9, 1.0))
        eye = torch.eye(2 * inner, dtype=torch.float64)
        want = plain.feed_forward(x, {"limit": 0.9}, {"gate": eye[:inner], "up": eye[inner:],
                                                       "down": torch.eye(inner, dtype=torch.float64)})
        assert float((out.double().cpu() - want).abs().max()) <= (2e-2 if dtype == torch.bfloat16 else 1e-6) * 2
    # The embedding with its position vector, into every stream.
    width, vocab = 36, 50
    table = rounded(torch.randn(vocab, width, generator=gen, dtype=torch.float64), dtype)
    ids, positions = [3, 49, 0, 7], [0, 1, 77, 1200]
    rates = torch.tensor([10000.0 ** (-2.0 * i / width) for i in range(width // 2)], dtype=torch.float64).float()
    streams = torch.empty((4, 3, width), dtype=torch.float32, device=device)
    i32 = lambda values: torch.tensor(values, dtype=torch.int32, device=device)
    ops.embedding_streams(i32(ids), table.to(dtype).to(device), i32(positions), rates.to(device), streams)
    want = table[ids] + plain.sinusoid(torch.tensor(positions), width)
    for s in range(3):
        assert float((streams[:, s].double().cpu() - want).abs().max()) <= 2e-4        # (an angle of 1200 in float32)
