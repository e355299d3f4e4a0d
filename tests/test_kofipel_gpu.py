"""Kofipel on the GPU: every new kernel alone against its torch stand-in and against the plain
implementation; inputs made so that one key decides (far back, at page borders, just inside and outside the
window and the kept keys, the sink); the engine against the plain model whole, with a decoded tail, in
portions down to two tokens and in mixed batches with pages and slots used again, in both precisions; long
decoding past the window; greedy generation through Engine.generate with and without graphs; the trace
program."""
import os
import types

import pytest
import torch

from tests import trace_tools as tt
from tests.kofipel_cases import CASES, make_folder
from tests.plain import kofipel_plain as plain
from tests.torch_ops import TorchOps

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from return_amd.kernels.hip_ops import HipOps
    return HipOps(DEV)


@pytest.fixture(scope="module")
def ref():
    return TorchOps(DEV)


def tol(dtype):
    return dict(atol=3e-5, rtol=3e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


def state_step(q_lens, slots, token_ids=None):
    cu = [0]
    for q in q_lens:
        cu.append(cu[-1] + q)
    return types.SimpleNamespace(n_seqs=len(q_lens), n_tokens=cu[-1], cu_q=i32(cu), slot_ids=i32(slots), cu_q_host=cu,
                                 slot_ids_host=list(slots), max_q_len=max(q_lens), token_ids=token_ids)


# ------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,taps,q_lens", [(10, 1, [5]), (72, 2, [1, 1, 1]), (300, 4, [1, 2, 3, 40, 17]),
                                          (4096, 4, [70]), (513, 8, [6, 7, 1, 30]), (64, 3, [1])])
@pytest.mark.parametrize("flags", [(True, False), (False, True)])
def test_causal_conv(ops, ref, dtype, C, taps, q_lens, flags):
    """Two steps in a row over slots that hold something: tails are read, results written, tails moved on;
    the input is a column slice of wider rows."""
    add_input, silu = flags
    n = len(q_lens)
    slots = torch.randperm(n + 2, generator=torch.Generator().manual_seed(n)).tolist()[:n]
    w = rnd(C, taps, seed=1, scale=0.5)
    tail_a = rnd(n + 2, taps - 1, C, dtype=dtype, seed=2)
    tail_b = tail_a.clone()
    for round_no in range(2):
        step = state_step(q_lens, slots)
        wide = rnd(sum(q_lens), C + 24, dtype=dtype, seed=3 + round_no)
        x = wide[:, 8:8 + C]
        a = torch.empty(sum(q_lens), C, dtype=dtype, device=DEV)
        b = torch.empty_like(a)
        ops.causal_conv(x, w, tail_a, step, a, add_input=add_input, silu=silu)
        ref.causal_conv(x, w, tail_b, step, b, add_input=add_input, silu=silu)
        torch.testing.assert_close(a.float(), b.float(), **tol(dtype))
        torch.testing.assert_close(tail_a.float(), tail_b.float(), atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,V,q_lens", [
    (4, 2, 16, 32, [1, 1, 1]), (3, 3, 12, 20, [5, 1, 33]), (2, 1, 64, 64, [40]), (6, 2, 20, 12, [2, 17]),
    (1, 1, 64, 48, [1, 19]), (2, 2, 128, 128, [1, 70]), (2, 1, 8, 256, [3]), (2, 2, 256, 16, [1, 4]), (5, 5, 7, 3, [9]),
    (1, 1, 384, 40, [2, 37]), (1, 1, 512, 8, [11]), (2, 2, 10, 100, [1, 40]), (2, 2, 100, 3, [37, 2]), (3, 3, 10, 100, [3]),
    (2, 2, 33, 10, [70]), (1, 1, 5, 200, [9, 1]), (1, 1, 80, 48, [33])])
def test_delta_rule(ops, ref, dtype, H, G, D, V, q_lens):
    """Two steps in a row over slots that hold something; the inputs are column slices of wider rows."""
    n = len(q_lens)
    T = sum(q_lens)
    slots = torch.randperm(n + 1, generator=torch.Generator().manual_seed(n)).tolist()[:n]
    qkv = rnd(T, 2 * G * D + H * V, dtype=dtype, seed=1)
    z = rnd(T, 24 + H, dtype=dtype, seed=2)
    ag = rnd(T, H * D + H * V + 8, dtype=dtype, seed=3)[:, :H * D + H * V]
    a_log, dt_bias, norm_w = rnd(H, seed=5), rnd(H * D, seed=6) - 1.0, 1 + rnd(V, seed=7, scale=0.1)
    state_a = rnd(n + 1, H, V, D, seed=8, scale=0.3)
    state_b = state_a.clone()
    for round_no in range(2):                                   # the second round starts from the first's state
        step = state_step(q_lens, slots)
        a = torch.empty(T, H * V, dtype=dtype, device=DEV)
        b = torch.empty_like(a)
        args = (qkv, z[:, 16:16 + H], ag, a_log, dt_bias, norm_w, 1e-5)
        ops.delta_rule(*args, state_a, step, a, H, G, D, V)
        ref.delta_rule(*args, state_b, step, b, H, G, D, V)
        torch.testing.assert_close(a.float(), b.float(), **tol(dtype))
        torch.testing.assert_close(state_a, state_b, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,H,S,with_delta", [(1, 72, 5, True), (7, 256, 24, False), (3, 4096, 64, True),
                                              (40, 1000, 17, True), (2, 8192, 33, False), (5, 64, 100, True),
                                              (301, 512, 16, True), (258, 4096, 32, False)])
def test_token_side(ops, ref, dtype, T, H, S, with_delta):
    table = rnd(50, 3 * S + 1, dtype=dtype, seed=1)
    gate, proj = rnd(S, H, dtype=dtype, seed=2, scale=H ** -0.5), rnd(H, S, dtype=dtype, seed=3)
    w = rnd(H, seed=4).abs()
    ids = torch.randint(0, 50, (T,), generator=torch.Generator().manual_seed(5)).int().to(DEV)
    delta = rnd(T, H, dtype=dtype, seed=6) if with_delta else None
    a = rnd(T, H, seed=7)
    b = a.clone()
    ops.token_side(a, delta, ids, table, S + 1, gate, proj, w, 1e-5)
    ref.token_side(b, delta, ids, table, S + 1, gate, proj, w, 1e-5)
    torch.testing.assert_close(a, b, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_relu_sq_and_bias(ops, ref, dtype):
    x = rnd(37, 333, dtype=dtype, seed=1)
    torch.testing.assert_close(ops.relu_sq(x.clone()).float(), ref.relu_sq(x.clone()).float(), **tol(dtype))
    b = rnd(333, seed=2)
    torch.testing.assert_close(ops.add_bias(x.clone(), b).float(), ref.add_bias(x.clone(), b).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,D,R,bias", [(4, 2, 16, 8, True), (3, 3, 24, 24, True), (6, 1, 12, 4, False),
                                             (2, 1, 128, 64, True), (5, 5, 40, 0, True), (2, 2, 320, 320, False)])
def test_qk_prepare_values_are_the_unrotated_keys(ops, ref, dtype, Hq, Hkv, D, R, bias):
    T, P, pages = 21, 8, 6
    qk = rnd(T, (Hq + Hkv) * D, dtype=dtype, seed=1)
    b = rnd((Hq + Hkv) * D, seed=2) if bias else None
    pos = torch.randint(0, 90, (T,), generator=torch.Generator().manual_seed(3)).int().to(DEV)
    ang = torch.outer(torch.arange(90).double(), 50.0 ** (-torch.arange(max(R // 2, 1)).double() / max(R // 2, 1)))
    cos, sin = ang.cos().float().to(DEV), ang.sin().float().to(DEV)
    slots = torch.randperm(pages * P, generator=torch.Generator().manual_seed(4))[:T].int().to(DEV)
    outs = []
    for o in (ops, ref):
        q = torch.zeros(T, Hq, D, dtype=dtype, device=DEV)
        kp = torch.zeros(pages, Hkv, P, D, dtype=dtype, device=DEV)
        vp = torch.zeros_like(kp)
        o.qk_prepare(qk, Hq, Hkv, D, b, pos, cos, sin, R, q, kp, vp, slots)
        outs.append((q, kp, vp))
    for a, b_ in zip(*outs):
        torch.testing.assert_close(a.float(), b_.float(), **tol(dtype))


def paged_step(q_lens, q_starts, P, pages_of):
    from tests.test_kernels_gpu import _step
    return _step(q_lens, q_starts, P, pages_of)


ATTN = [  # Hq, Hkv, D, P, [(q_len, q_start)], window, keep_first, softcap
    (4, 2, 16, 16, [(5, 0), (17, 0), (33, 0)], 0, 0, 0.0),
    (4, 2, 64, 16, [(1, 300), (1, 5), (1, 64)], 136, 20, 20.0),
    (6, 1, 32, 8, [(24, 100), (1, 0), (2, 62), (1, 399)], 33, 40, 4.0),
    (3, 3, 24, 16, [(70, 0), (1, 130), (40, 90)], 9, 0, 0.0),
    (2, 1, 128, 16, [(130, 200)], 70, 3, 50.0),
    (5, 5, 48, 32, [(1, 1000), (3, 997)], 64, 64, 2.0),
    (8, 2, 20, 4, [(1, 77), (19, 58)], 5, 1, 0.0),
    (4, 2, 64, 16, [(1, 300), (1, 90), (1, 2000)], 0, 0, 10.0),       # no window: a request's splits may be merged in one workgroup
    (16, 2, 128, 16, [(1, 700), (1, 64), (1, 1), (1, 5000)], 1024, 64, 30.0),
    (16, 2, 128, 16, [(1, 1500), (300, 1200), (1, 8)], 128, 64, 30.0),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,D,P,segs,window,keep,cap", ATTN)
def test_attention_with_kept_keys_cap_temperature_and_sink(ops, ref, dtype, Hq, Hkv, D, P, segs, window, keep, cap,
                                                           monkeypatch):
    if window == 0:
        monkeypatch.setattr(ops, "decode_merge_round", 1)         # (the merge inside the workgroup, where it applies)
    q_lens, q_starts = [s[0] for s in segs], [s[1] for s in segs]
    need = [-(-(a + b) // P) for a, b in segs]
    perm = torch.randperm(sum(need) + 3, generator=torch.Generator().manual_seed(5)).tolist()
    pages_of = [[perm.pop() for _ in range(k)] for k in need]
    step = paged_step(q_lens, q_starts, P, pages_of)
    kp = rnd(sum(need) + 3, Hkv, P, D, dtype=dtype, seed=51)
    vp = rnd(sum(need) + 3, Hkv, P, D, dtype=dtype, seed=52)
    q = rnd(sum(q_lens), Hq, D, dtype=dtype, seed=53)
    temp = (1 + rnd(Hq, seed=54, scale=0.2)).abs()
    a, b = torch.zeros_like(q), torch.zeros_like(q)
    kw = dict(head_scale=temp, softcap=cap, keep_first=keep, sink=True)
    ops.attention(q, a, kp, vp, step, 0, 0.3, window, **kw)
    ref.attention(q, b, kp, vp, step, 0, 0.3, window, **kw)
    torch.testing.assert_close(a.float(), b.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_len", [1, 2, 7, 70])
@pytest.mark.parametrize("where", ["window_in", "window_out", "kept_in", "kept_out", "far_kept", "page_border"])
def test_attention_one_key_decides(ops, dtype, q_len, where):
    """All scores are 0 but one key's, which is large: if the last query may read that key its output is that
    key's value, else it is the sum of the values it reads over their number plus one, the sink's share. The
    key sits just inside or outside the window, just inside or outside the kept keys, far back among hundreds,
    or on a page's last row; pages lie scattered; one token goes the decode way, several the prompt's."""
    Hq, Hkv, D, P, window, keep = 4, 2, 64, 16, 37, 19
    L = 431
    last = L - 1
    spot = {"window_in": last - window + 1, "window_out": last - window, "kept_in": keep - 1, "kept_out": keep,
            "far_kept": 2, "page_border": last - 21 - (last - 21) % P + P - 1}[where]
    seen = where not in ("window_out", "kept_out")
    start = L - q_len
    n_pages = -(-L // P)
    perm = torch.randperm(n_pages + 4, generator=torch.Generator().manual_seed(9)).tolist()
    pages = perm[:n_pages]
    step = paged_step([q_len], [start], P, [pages])
    k = torch.zeros(L, Hkv, D)
    k[spot, :, 0] = 64.0
    v = rnd(L, Hkv, D, seed=71).cpu()
    kp = torch.zeros(n_pages + 4, Hkv, P, D)
    vp = torch.zeros_like(kp)
    for i in range(L):
        kp[pages[i // P], :, i % P] = k[i]
        vp[pages[i // P], :, i % P] = v[i]
    kp, vp = kp.to(dtype).to(DEV), vp.to(dtype).to(DEV)
    q = torch.zeros(q_len, Hq, D)
    q[:, :, 0] = 1.0
    q = q.to(dtype).to(DEV)
    out = torch.zeros_like(q)
    ops.attention(q, out, kp, vp, step, 0, 0.5, window, head_scale=torch.ones(Hq, device=DEV), softcap=30.0,
                  keep_first=keep, sink=True)
    vv = v.to(dtype).double()
    if seen:
        want = vv[spot]                                       # exp(30 tanh(32/30)) against a few dozen ones
        atol = 2e-2 if dtype == torch.bfloat16 else 1e-4
    else:
        read = [j for j in range(L) if j < keep or last - j < window]
        assert spot not in read
        want = vv[read].sum(0) / (len(read) + 1)
        atol = 1e-2 if dtype == torch.bfloat16 else 1e-5
    got = out[q_len - 1].double().cpu()
    torch.testing.assert_close(got, want.repeat_interleave(Hq // Hkv, dim=0), atol=atol, rtol=0,
                               msg=lambda m: f"key {spot} ({where}), query at {last}: {m}")


# ------------------------------------------------------------------ the engine against the plain model
LENGTHS = {"a": 5, "b": 17, "c": 33, "d": 100, "e": 64, "f": 150, "g": 1, "h": 47}
# A row's error: the root mean square over the vocabulary of the difference of the logits, its mean taken off,
# over the root mean square of the plain logits. 32-bit: ten times the largest seen on these traces (3e-6).
# bfloat16: what rounding alone does differs from row to row by a factor of ten (a stand-in engine of torch
# operations that rounds where the kernels round is 0.01 to 0.14 away from the plain logits on the very rows
# on which the kernels are), so the kernels are held against that stand-in, row by row (twice the largest
# difference seen, 0.04), and against the plain logits on average and by a bound that only a fault exceeds.
ROW_ERROR = {"float32": 5e-5, "bfloat16": 0.3}
ROW_ERROR_16_MEAN = 0.03
ROW_ERROR_16_STAND_IN = 0.08


@pytest.fixture(scope="module", params=sorted(CASES))
def model(request, tmp_path_factory):
    folder = make_folder(tmp_path_factory, request.param)
    cfg, w = plain.read_folder(folder)
    reqs = {rid: tt.random_tokens(cfg["vocab"], n, seed=ord(rid)) for rid, n in LENGTHS.items()}
    want = {rid: plain.logits(cfg, w, toks) for rid, toks in reqs.items()}
    # the same requests, whole, through the engine with torch operations in bfloat16 in place of the kernels
    steps = tt.whole(reqs)
    rounded = tt.run_in_process(make_runner(folder, "bfloat16", tt.peak_tokens(steps), ops=TorchOps(DEV)), steps)
    return folder, cfg, reqs, want, rounded


def make_runner(folder, dtype, max_tokens, page=16, ops=None, **kw):
    from return_amd.config import EngineConfig
    from return_amd.engine import ModelRunner
    ec = EngineConfig(dtype=dtype, page_size=page, max_token=max_tokens, max_reside=4, max_step_tokens=max(max_tokens, 4),
                      prefill_chunk=max_tokens, tune_products=False, check_invariants=True, **kw)
    return ModelRunner(folder, engine_config=ec, ops=ops)


def row_error(a, b):
    d = (a - b).double()
    return float((d - d.mean()).pow(2).mean().sqrt() / b.double().pow(2).mean().sqrt())


def compare(got, want, reqs, dtype, rounded=None):
    worst, total, n = 0.0, 0.0, 0
    for rid, toks in reqs.items():
        for p in range(len(toks)):
            e = row_error(got[(rid, p)], want[rid][p])
            worst, total, n = max(worst, e), total + e, n + 1
            assert e <= ROW_ERROR[dtype], f"request {rid} position {p} (first wrong place): row error {e:.3e}"
            if dtype == "float32":
                assert int(got[(rid, p)].argmax()) == int(want[rid][p].argmax()), f"request {rid} position {p}: argmax"
            elif rounded is not None:
                e16 = row_error(got[(rid, p)], rounded[(rid, p)])
                assert e16 <= ROW_ERROR_16_STAND_IN, \
                    f"request {rid} position {p} (first wrong place): {e16:.3e} from the stand-in that rounds alike"
    if dtype == "bfloat16":
        assert total / n <= ROW_ERROR_16_MEAN, f"mean row error {total / n:.3e}"
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "tail_decoded", "portions", "mixed"])
def test_engine_matches_plain(model, dtype, cut):
    folder, cfg, reqs, want, rounded = model
    steps = {"whole": tt.whole, "tail_decoded": tt.tail_decoded, "portions": tt.portions, "mixed": tt.mixed}[cut](reqs)
    runner = make_runner(folder, dtype, tt.peak_tokens(steps))
    got = tt.run_in_process(runner, steps)
    print(f"kofipel {dtype} {cut}: largest row error {compare(got, want, reqs, dtype, rounded):.2e}")
    assert not runner.cache.live and all(g.pages.in_use() == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_passes_the_window(tmp_path_factory, dtype):
    """A short prompt and 280 tokens one by one: the windows (70 and 20 keys) pass over decoded tokens only,
    the kept keys stay, the delta rule's state is carried through every step."""
    folder = make_folder(tmp_path_factory, "a")
    cfg, w = plain.read_folder(folder)
    toks = tt.random_tokens(cfg["vocab"], 300, seed=4)
    steps = tt.tail_decoded({"r": toks}, tail=280)
    got = tt.run_in_process(make_runner(folder, dtype, 320), steps)
    print(f"kofipel {dtype} long decoding: largest row error {compare(got, {'r': plain.logits(cfg, w, toks)}, {'r': toks}, dtype):.2e}")


def test_batches_of_unequal_requests_equal_each_alone(tmp_path_factory):
    """A request's logits do not depend on what else is in the step, beyond the rounding of products that
    the library forms in another order for another number of rows."""
    folder = make_folder(tmp_path_factory, "b")
    cfg, _ = plain.read_folder(folder)
    reqs = {rid: tt.random_tokens(cfg["vocab"], n, seed=ord(rid)) for rid, n in (("a", 70), ("b", 3), ("c", 41), ("d", 1))}
    sizes = {"a": [30, 1, 1, 38], "b": [1, 2], "c": [2, 39], "d": [1]}
    alone = {}
    for rid, toks in reqs.items():
        r = make_runner(folder, "float32", 256)
        alone.update(tt.run_in_process(r, tt.portions({rid: toks}, sizes=tuple(sizes[rid]))))
    steps, at = [], {rid: 0 for rid in reqs}
    for k in range(4):
        entries, end = [], []
        for rid, toks in reqs.items():
            if k < len(sizes[rid]):
                n = sizes[rid][k]
                entries.append({"id": rid, "tokens": toks[at[rid]:at[rid] + n], "want": list(range(n))})
                at[rid] += n
                if at[rid] == len(toks):
                    end.append(rid)
        steps.append({"step": k, "entries": entries, "end": end})
    together = tt.run_in_process(make_runner(folder, "float32", 256), steps)
    for key, row in alone.items():
        assert row_error(together[key], row) < 2e-5


# ------------------------------------------------------------------ generation and the programs
def test_greedy_generation_through_the_engine(tmp_path_factory):
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    for name in ("a", "b"):
        folder = make_folder(tmp_path_factory, name)
        cfg, w = plain.read_folder(folder)
        prompts = [tt.random_tokens(cfg["vocab"], n, seed=n) for n in (1, 8, 31, 64, 90)]
        want = [plain.greedy(cfg, w, p, 12) for p in prompts]
        for graphs in (False, True):
            eng = Engine(folder, dtype="float32", page_size=16, max_token=1024, max_reside=4, max_step_tokens=64,
                         prefill_chunk=24, use_graphs=graphs, check_invariants=True)
            got = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12))
            assert [r.output_ids for r in got] == want, f"model {name}, graphs {graphs}"
            assert not eng.runner.cache.live


def test_bf16_generation_from_graphs_equals_eager(tmp_path_factory):
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    folder = make_folder(tmp_path_factory, "a")
    cfg, _ = plain.read_folder(folder)
    prompts = [tt.random_tokens(cfg["vocab"], n, seed=n) for n in (3, 40, 77)]
    outs = []
    for graphs in (False, True):
        eng = Engine(folder, dtype="bfloat16", page_size=16, max_token=1024, max_reside=4, use_graphs=graphs)
        outs.append([r.output_ids for r in eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=24))])
    assert outs[0] == outs[1]


def test_trace_program_on_a_model_folder(tmp_path_factory, tmp_path):
    folder = make_folder(tmp_path_factory, "b")
    cfg, w = plain.read_folder(folder)
    reqs = {rid: tt.random_tokens(cfg["vocab"], n, seed=ord(rid)) for rid, n in (("a", 40), ("b", 7), ("c", 90))}
    steps = tt.mixed(reqs, seed=3, max_live=3)
    got = tt.run_program(folder, "float32", steps, str(tmp_path), tt.peak_tokens(steps), cfg["vocab"],
                         env=dict(os.environ))
    compare(got, {rid: plain.logits(cfg, w, t) for rid, t in reqs.items()}, reqs, "float32")
