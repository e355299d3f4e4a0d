"""Rupezen on the CPU: configuration, spec and tensor names, the torch stand-ins of its kernels against the
plain implementation mechanism by mechanism, the cache manager's chunks and pools of two widths, and the
engine's host side (cache manager, step function, looped layers with their pass input, slots and pages
that are used again) against the plain model under every cut."""
import copy
import types

import pytest
import torch

from tests import trace_tools as tt
from tests.plain import rupezen_plain as plain
from tests.rupezen_cases import CASES, RUPE_A, RUPE_B, make_folder
from tests.torch_ops import TorchOps


@pytest.fixture(scope="module", params=sorted(CASES))
def model(request, tmp_path_factory):
    folder = make_folder(tmp_path_factory, request.param)
    cfg, w = plain.read_folder(folder)
    return folder, cfg, w


def runner_for(folder, max_tokens, page=16, max_live=4, **kw):
    from return_amd.config import EngineConfig
    from return_amd.engine import ModelRunner
    ec = EngineConfig(dtype="float32", device="cpu", page_size=page, max_token=max_tokens, max_reside=max_live,
                      max_step_tokens=max(max_tokens, 4), prefill_chunk=max_tokens, use_graphs=False,
                      tune_products=False, **kw)
    return ModelRunner(folder, engine_config=ec, ops=TorchOps("cpu"))


# ------------------------------------------------------------------ configuration and spec
def test_config_reads_every_layer_and_refuses_what_it_cannot_run():
    from return_amd.config.base import ConfigError
    from return_amd.config.rupezen import RupezenConfig
    cfg = RupezenConfig.from_dict(RUPE_A)
    assert cfg.run_order() == [(0, 0, False), (1, 0, True), (2, 0, False), (1, 1, True), (2, 1, False), (3, 0, False)]
    assert RupezenConfig.from_dict(RUPE_B).run_order() == [(i, 0, False) for i in range(3)]
    assert RupezenConfig.from_dict(cfg.to_dict()) == cfg
    for change in (lambda c: c["layers"][0].update(type="convolution"),
                   lambda c: c["layers"][0]["mixer"].update(kv_heads=3),
                   lambda c: c["layers"][0]["mixer"].pop("diff"),
                   lambda c: c["layers"][0]["mixer"]["rot"].update(dims=3),
                   lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10),
                   lambda c: c["layers"][0]["mlp"].update(kind="dense"),
                   lambda c: c["layers"][0]["mlp"]["router"].update(top=5),
                   lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=3),
                   lambda c: c["loop"].update(stop=9),
                   lambda c: c.pop("norm")):
        bad = copy.deepcopy(RUPE_A)
        change(bad)
        with pytest.raises(ConfigError):
            RupezenConfig.from_dict(bad)


def test_spec_names_the_tensors_and_gives_every_pass_its_own_cache(model):
    from return_amd.config import load_config, lookup_architecture
    folder, cfg, w = model
    config = load_config(folder)
    spec = lookup_architecture(config.architecture)[1](config)
    assert set(spec.expected_tensors()) == set(w)
    layers = [call.cache for call in spec.schedule]
    assert len(layers) == len(set(layers))
    order, _ = plain.run_order(cfg)
    assert [call.block for call in spec.schedule] == [i for i, _, _ in order]
    assert [call.pass_input for call in spec.schedule] == \
        [p if (cfg.get("loop") and first) else None for _, p, first in order]
    assert (spec.pass_input is not None) == bool(cfg.get("loop"))
    assert spec.head.tensors["weight"] == spec.embedding.tensors["weight"]


# ------------------------------------------------------------------ the cache manager: chunks and two widths
def test_chunked_layers_give_pages_back_at_the_chunk_border_and_pools_have_two_widths():
    from return_amd.cache import CacheManager
    from return_amd.cache.spec import PagedKVSpec
    P = 4
    cm = CacheManager({0: PagedKVSpec(2, 6, None, 0, 10, 10), 1: PagedKVSpec(1, 8, None, 0, None, None)}, P, 64, 2,
                      torch.float32)
    chunked = cm.group_of[0]
    view = cm.view(0)
    assert tuple(view.k_pool.shape) == (17, 2, P, 6) and tuple(view.v_pool.shape) == (17, 2, P, 10)
    assert cm.view(1).k_pool.shape == cm.view(1).v_pool.shape
    cm.add_request("r")
    held = []
    for n in (9, 1, 1, 8, 1, 1, 30):
        tables = cm.begin_step([("r", n)])
        g = tables.groups[chunked]
        first_new = int(tables.q_start[0])
        # every key that a token of this step reads is on a listed page
        assert int(g.kv_start[0]) <= first_new // 10 * 10
        cm.end_step()
        cm.check_invariants()
        r = cm.live["r"]
        assert r.first_pos[chunked] <= r.seq_len // 10 * 10 < r.first_pos[chunked] + P + (len(r.pages[chunked]) * P or 1)
        held.append(len(r.pages[chunked]))
    assert max(held) <= cm.max_pages(64, 30)[chunked]
    assert cm.live["r"].first_pos[chunked] == 48            # 51 tokens: the chunk from 50 on, pages from 48
    assert len(cm.live["r"].pages[cm.group_of[1]]) == 13     # the other layer keeps everything
    cm.free_request("r")
    assert all(grp.pages.in_use() == 0 for grp in cm.groups)


# ------------------------------------------------------------------ the stand-ins, mechanism by mechanism
def _attention_weights(g, W, H, G, D, V):
    w = {"q": torch.randn(H * 2 * D, W, generator=g), "k": torch.randn(G * 2 * D, W, generator=g),
         "v": torch.randn(G * V, W, generator=g), "o": torch.eye(H * V),
         "lq1": 0.3 * torch.randn(D, generator=g), "lk1": 0.3 * torch.randn(D, generator=g),
         "lq2": 0.3 * torch.randn(D, generator=g), "lk2": 0.3 * torch.randn(D, generator=g)}
    return {k: v.double() for k, v in w.items()}


def run_attention_in_pieces(ops, h, w, m, eps, pieces, P=16, pages=(2, 0, 3, 1), dtype=torch.float32, device="cpu"):
    """One layer's differential attention through maps_qkv_prepare and attention_diff of a kernel set, the
    sequence cut into the given pieces, on pages in a shuffled order."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    R = m["rot"]["dims"] if m.get("rot") else 0
    chunk = m["mask"]["size"] if m.get("mask") else 0
    qkv = torch.cat([h @ w["q"].T, h @ w["k"].T, h @ w["v"].T], dim=1).to(dtype).to(device)
    cos = sin = None
    if R:
        ang = torch.outer(torch.arange(T).double(), m["rot"]["base"] ** (-torch.arange(R // 2).double() * 2 / R))
        cos, sin = ang.cos().float().to(device), ang.sin().float().to(device)
    lam = plain.differential_lambda(w, "", m["diff"])
    kp = torch.zeros(len(pages), G, P, 2 * D, dtype=dtype, device=device)
    vp = torch.zeros(len(pages), G, P, V, dtype=dtype, device=device)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    out, at = torch.empty(T, H, V, dtype=dtype, device=device), 0
    for n in pieces:
        pos = list(range(at, at + n))
        slots = i32([pages[p // P] * P + p % P for p in pos])
        grp = types.SimpleNamespace(page_table=i32(list(pages)), cu_pages=i32([0, len(pages)]), kv_start=i32([0]))
        tiles = {} if n == 1 else {64: i32([[0, off] for off in range(0, n, 64)])}      # q tiles, for a kernel that reads them
        step = types.SimpleNamespace(groups=[grp], n_seqs=1, n_tokens=n, cu_q=i32([0, n]), q_start=i32([at]),
                                     n_decode=1 if n == 1 else 0, prefill_tiles=tiles, q_lens=[n], q_starts=[at],
                                     n_prefill_tokens=0 if n == 1 else n, decode_segs=None, prefill_toks=None,
                                     max_decode_seq_len=at + n if n == 1 else 0)
        q = torch.empty(n, H, 2 * D, dtype=dtype, device=device)
        ops.maps_qkv_prepare(qkv[at:at + n].contiguous(), H, G, 2, D, V, i32(pos), cos, sin, R, True, q, kp, vp, slots)
        o = torch.empty(n, H, V, dtype=dtype, device=device)
        ops.attention_diff(q, o, kp, vp, step, 0, m["scale"], lam, eps, 1.0 - m["diff"], window=0, chunk=chunk)
        out[at:at + n] = o
        at += n
    assert at == T
    return out.reshape(T, H * V)


@pytest.mark.parametrize("sizes", [(4, 2, 8, 12, 20, 4), (3, 3, 6, 7, None, 6), (2, 1, 10, 32, 16, 0)])
def test_attention_stand_in_in_pieces_equals_the_plain_function(sizes):
    H, G, D, V, chunk, R = sizes
    g = torch.Generator().manual_seed(H * 100 + D)
    T, W = 53, 24
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.6, "diff": 0.35}
    if chunk:
        m["mask"] = {"size": chunk}
    if R:
        m["rot"] = {"base": 100.0, "dims": R}
    w = _attention_weights(g, W, H, G, D, V)
    h = torch.randn(T, W, generator=g).double()
    want = plain.differential_attention(h, w, "", m, 1e-5)
    got = run_attention_in_pieces(TorchOps("cpu"), h, w, m, 1e-5, (7, 1, 1, 13, 2, 1, 20, 8))
    torch.testing.assert_close(got.double(), want, atol=3e-5, rtol=1e-4)


def test_a_key_just_outside_the_chunk_is_not_read_and_one_just_inside_is():
    """One key is made to decide a query's first map; the plain function sees it only from inside the chunk."""
    g = torch.Generator().manual_seed(3)
    W, H, G, D, V, C = 16, 2, 1, 8, 8, 10
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 1.0, "diff": 0.5, "mask": {"size": C}}
    w = _attention_weights(g, W, H, G, D, V)
    h = 0.1 * torch.randn(27, W, generator=g).double()
    h[19] *= 60.0                                      # the last key of the second chunk: large k and v
    h[20] = h[19]                                      # the first query of the third chunk looks its way
    h[18] = h[19] / 60.0 * 55.0                        # and so does one inside the second chunk
    want = plain.differential_attention(h, w, "", m, 1e-6)
    for pieces in ((27,), (19, 1, 1, 6), (20, 7), (18, 2, 2, 5)):
        got = run_attention_in_pieces(TorchOps("cpu"), h, w, m, 1e-6, pieces)
        torch.testing.assert_close(got.double(), want, atol=1e-4, rtol=1e-4)
    # the check has teeth: without the chunk the query at 20 reads the key at 19
    m_open = dict(m)
    m_open.pop("mask")
    assert (plain.differential_attention(h, w, "", m_open, 1e-6)[20] - want[20]).abs().max() > 0.1


@pytest.mark.parametrize("E,top,count,keep", [(8, 2, 4, 2), (6, 3, 2, 1), (5, 1, 1, 1), (6, 2, 6, 3), (9, 4, 3, 2), (4, 4, 1, 1)])
def test_router_stand_in_equals_the_plain_choice(E, top, count, keep):
    g = torch.Generator().manual_seed(E * 10 + top)
    z = 2.0 * torch.randn(40, E, generator=g)
    corr = 0.5 * torch.randn(E, generator=g)
    want_ids, want_w = plain.route(z.double(), corr.double(), top, count, keep)
    ids, w = TorchOps("cpu").moe_route(z, corr, top, count, keep, 1e-20)
    assert ids.long().tolist() == want_ids.tolist()
    torch.testing.assert_close(w.double(), want_w, atol=1e-6, rtol=1e-5)
    # the correction steers the choice but not the weights: they are the chosen sigmoids over their sum
    torch.testing.assert_close(w.sum(-1), torch.ones(40), atol=1e-5, rtol=0)


def test_a_group_that_is_left_out_gives_no_expert_even_with_the_largest_score():
    """Experts 0, 1 form a group with one very large and one very small score; the other group's two are both
    fairly large and win on the sum of two, so the single largest expert is not chosen."""
    z = torch.tensor([[6.0, -9.0, 2.0, 2.1]])
    ids, _ = plain.route(z.double(), torch.zeros(4).double(), 2, 2, 1)
    assert sorted(ids[0].tolist()) == [2, 3]
    got, _ = TorchOps("cpu").moe_route(z, torch.zeros(4), 2, 2, 1, 1e-20)
    assert sorted(got[0].tolist()) == [2, 3]
    # choice scores below zero: an expert of a kept group still beats every expert of a group that is left out
    # (were the others' scores set to 0 instead, they would win over these negative ones)
    z = torch.tensor([[-2.0, -2.1, -1.5, -8.0]])
    corr = torch.tensor([-1.0, -1.0, -1.0, -1.0])
    ids, _ = plain.route(z.double(), corr.double(), 2, 2, 1)
    got, _ = TorchOps("cpu").moe_route(z, corr, 2, 2, 1, 1e-20)
    assert sorted(ids[0].tolist()) == sorted(got[0].tolist()) == [0, 1]


def test_experts_stand_in_equals_the_plain_feed_forward():
    g = torch.Generator().manual_seed(8)
    T, W, I, E, top = 9, 12, 10, 6, 3
    w = {"router": torch.randn(E, W, generator=g), "correction": 0.3 * torch.randn(E, generator=g)}
    for e in range(E):
        w.update({f"e{e}.gate": torch.randn(I, W, generator=g), f"e{e}.up": torch.randn(I, W, generator=g),
                  f"e{e}.down": torch.randn(W, I, generator=g)})
    w = {k: v.double() for k, v in w.items()}
    mlp = {"expert": {"ff": I}, "router": {"experts": E, "top": top, "groups": {"count": 3, "keep": 2}}}
    h = torch.randn(T, W, generator=g).double()
    want = plain.routed_feed_forward(h, w, "", mlp)
    ops = TorchOps("cpu")
    ids, weights = ops.moe_route((h @ w["router"].T).float(), w["correction"].float(), top, 3, 2, 1e-20)
    gate_up = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(E)]).float()
    down = torch.stack([w[f"e{e}.down"] for e in range(E)]).float()
    got = ops.moe_experts(h.float(), ids, weights, gate_up, down)
    torch.testing.assert_close(got.double(), want, atol=2e-4, rtol=1e-4)


def test_pass_input_and_scaled_sublayers():
    """h <- W [h + m pending ; h0] + step[t], and a norm that adds m times what is pending."""
    from return_amd.parts.norm import RMSNorm
    from return_amd.parts.passes import ConcatLinearPassInput
    from return_amd.parts.runtime import Runtime, Scaled
    g = torch.Generator().manual_seed(4)
    T, W = 5, 12
    rt = Runtime("cpu", "float32", ops=TorchOps("cpu"))
    wt = {"weight": torch.randn(W, 2 * W, generator=g), "step": torch.randn(3, W, generator=g)}
    part = ConcatLinearPassInput({"hidden_size": W, "passes": 3}, wt, rt)
    h, h0, d = (torch.randn(T, W, generator=g) for _ in range(3))
    want = torch.cat([h + 0.3 * d, h0], dim=1) @ wt["weight"].T + wt["step"][2]
    got, pending = part.forward(h.clone(), Scaled(d, 0.3), h0, 2)
    assert pending is None
    torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)
    with pytest.raises(ValueError):
        part.forward(h.clone(), None, h0, 3)
    norm = RMSNorm({"size": W, "eps": 1e-5}, {"weight": torch.rand(W, generator=g) + 0.5}, rt)
    hh = h.clone()
    y = norm.forward(hh, Scaled(d, 0.3))
    torch.testing.assert_close(hh, h + 0.3 * d)
    torch.testing.assert_close(y.double(), plain.rms_norm((h + 0.3 * d).double(), norm.weight.double(), 1e-5).double(),
                               atol=1e-5, rtol=1e-5)


# ------------------------------------------------------------------ the engine's host side against the plain model
LENGTHS = {"a": 5, "b": 17, "c": 33, "d": 100, "e": 64, "f": 131, "g": 1, "h": 47}


def test_layers_one_by_one_against_the_plain_model(model):
    """The stream after every layer run, a looped layer each time."""
    from return_amd.engine.runner import StepEntry
    from return_amd.parts.runtime import unscaled
    folder, cfg, w = model
    runner = runner_for(folder, 64)
    seen = []
    for block in runner.model.blocks:
        def wrap(f=block.forward):
            def run(h, pending, *a, **k):
                h2, p2 = f(h, pending, *a, **k)
                d, factor = unscaled(p2)
                seen.append(h2 + factor * d.float())
                return h2, p2
            return run
        block.forward = wrap()
    toks = tt.random_tokens(cfg["vocab"], 37, seed=5)
    runner.add_request("r")
    runner.step([StepEntry("r", toks, [0])])
    want, _ = plain.hidden_states(cfg, w, toks)
    assert len(seen) == want.shape[0]
    for run, (got, ref) in enumerate(zip(seen, want)):
        torch.testing.assert_close(got.double(), ref, atol=2e-4, rtol=1e-4, msg=lambda m: f"layer run {run}: {m}")


@pytest.mark.parametrize("cut", ["whole", "tail_decoded", "portions", "mixed"])
def test_engine_matches_plain_under_every_cut(model, cut):
    folder, cfg, w = model
    reqs = {rid: tt.random_tokens(cfg["vocab"], n, seed=ord(rid)) for rid, n in LENGTHS.items()}
    steps = {"whole": tt.whole, "tail_decoded": tt.tail_decoded, "portions": tt.portions, "mixed": tt.mixed}[cut](reqs)
    # the pool holds exactly the trace's peak and there are four slots: pages and slots are used again
    runner = runner_for(folder, tt.peak_tokens(steps), check_invariants=True)
    got = tt.run_in_process(runner, steps)
    for rid, toks in reqs.items():
        want = plain.logits(cfg, w, toks)
        for p in range(len(toks)):
            torch.testing.assert_close(got[(rid, p)].double(), want[p], atol=3e-4, rtol=1e-4,
                                       msg=lambda m: f"request {rid} position {p} (first wrong place): {m}")
    assert not runner.cache.live and all(g.pages.in_use() == 0 for g in runner.cache.groups)


def test_a_request_that_takes_over_pages_does_not_see_what_was_left(tmp_path_factory):
    folder = make_folder(tmp_path_factory, "b")
    cfg, w = plain.read_folder(folder)
    runner = runner_for(folder, 128, max_live=1)
    first = tt.random_tokens(cfg["vocab"], 90, seed=1)
    second = tt.random_tokens(cfg["vocab"], 30, seed=2)
    tt.run_in_process(runner, tt.whole({"x": first}))
    got = tt.run_in_process(runner, tt.portions({"y": second}, sizes=(2, 3, 1, 9)))
    want = plain.logits(cfg, w, second)
    for p in range(len(second)):
        torch.testing.assert_close(got[("y", p)].double(), want[p], atol=3e-4, rtol=1e-4)
