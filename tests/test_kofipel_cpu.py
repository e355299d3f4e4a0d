"""Kofipel on the CPU: configuration, spec and tensor names, the torch stand-ins of its kernels against the
plain implementation mechanism by mechanism, and the engine's host side (cache and state manager, step
function, looped layers, slots and pages that are used again) against the plain model under every cut."""
import copy

import pytest
import torch

from tests import trace_tools as tt
from tests.kofipel_cases import CASES, KOFI_A, KOFI_B, make_folder
from tests.plain import kofipel_plain as plain
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
    from return_amd.config.kofipel import KofipelConfig
    cfg = KofipelConfig.from_dict(KOFI_A)
    assert cfg.run_order() == [(0, 0), (1, 0), (2, 0), (1, 1), (2, 1), (3, 0)]
    assert KofipelConfig.from_dict(KOFI_B).run_order() == [(i, 0) for i in range(4)]
    assert KofipelConfig.from_dict(cfg.to_dict()) == cfg
    for change in (lambda c: c["layers"][0].update(type="convolution"),
                   lambda c: c["layers"][1]["mixer"].update(kv_heads=3),
                   lambda c: c["layers"][1]["mixer"].update(vdim=8),
                   lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7),
                   lambda c: c["layers"][0]["mlp"].update(kind="routed"),
                   lambda c: c["loop"].update(stop=9),
                   lambda c: c.pop("norm")):
        bad = copy.deepcopy(KOFI_A)
        change(bad)
        with pytest.raises(ConfigError):
            KofipelConfig.from_dict(bad)


def test_spec_names_the_tensors_and_gives_every_pass_its_own_cache(model):
    from return_amd.config import load_config, lookup_architecture
    folder, cfg, w = model
    config = load_config(folder)
    spec = lookup_architecture(config.architecture)[1](config)
    assert set(spec.expected_tensors()) == set(w)
    layers = [c for call in spec.schedule for c in (call.cache if isinstance(call.cache, tuple) else (call.cache,))]
    assert len(layers) == len(set(layers))
    assert [call.block for call in spec.schedule] == [i for i, _ in plain.run_order(cfg)]
    starts = [call.add_input for call in spec.schedule]
    want = [bool(cfg.get("loop")) and p > 0 and i == cfg["loop"]["start"] for i, p in plain.run_order(cfg)]
    assert starts == want


def test_a_stored_model_gives_the_rank_of_its_low_rank_maps(tmp_path_factory):
    """config.json need not name the rank: the shapes in the file do."""
    import json
    import os
    folder = make_folder(tmp_path_factory, "a")
    path = os.path.join(folder, "config.json")
    with open(path) as f:
        raw = json.load(f)
    for layer in raw["layers"]:
        layer["mixer"].pop("rank", None)
    with open(path, "w") as f:
        json.dump(raw, f)
    cfg, w = plain.read_folder(folder)
    toks = tt.random_tokens(cfg["vocab"], 12, seed=3)
    got = tt.run_in_process(runner_for(folder, 64), tt.whole({"r": toks}))
    torch.testing.assert_close(torch.stack([got[("r", p)] for p in range(12)]), plain.logits(cfg, w, toks),
                               atol=2e-4, rtol=1e-4)


# ------------------------------------------------------------------ the stand-ins, mechanism by mechanism
class _Step:
    def __init__(self, q_lens, slots, token_ids=None):
        self.n_seqs, self.n_tokens = len(q_lens), sum(q_lens)
        self.cu_q_host = [0]
        for q in q_lens:
            self.cu_q_host.append(self.cu_q_host[-1] + q)
        self.slot_ids_host = list(slots)
        self.max_q_len = max(q_lens)
        self.token_ids = token_ids


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_convolution_in_pieces_equals_the_whole(taps):
    g = torch.Generator().manual_seed(taps)
    T, C = 23, 10
    x = torch.randn(T, C, generator=g)
    w = torch.randn(C, taps, generator=g)
    want = x.double() + plain.causal_filter(x.double(), w.double())
    ops = TorchOps("cpu")
    tail = torch.randn(3, taps - 1, C, generator=g)             # slots hold what an earlier request left
    tail[1].zero_()                                             # (a new request's slot is cleared)
    got, at = [], 0
    for n in (1, 2, 1, 5, 1, 13):
        out = torch.empty(n, C)
        ops.causal_conv(x[at:at + n], w, tail, _Step([n], [1]), out, add_input=True)
        got.append(out)
        at += n
    torch.testing.assert_close(torch.cat(got).double(), want, atol=1e-5, rtol=1e-5)


def test_delta_rule_in_pieces_equals_the_plain_recurrence():
    g = torch.Generator().manual_seed(5)
    T, W, H, G, D, V, r = 19, 24, 4, 2, 6, 10, 3
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V}
    w = {"q": torch.randn(G * D, W, generator=g), "k": torch.randn(G * D, W, generator=g),
         "v": torch.randn(H * V, W, generator=g), "q.conv": torch.zeros(G * D, 1) + 1, "k.conv": torch.zeros(G * D, 1) + 1,
         "v.conv": torch.zeros(H * V, 1) + 1, "b": torch.randn(H, W, generator=g), "A_log": torch.randn(H, generator=g),
         "dt_bias": torch.randn(H * D, generator=g), "norm": 1 + 0.1 * torch.randn(V, generator=g),
         "a1": torch.randn(r, W, generator=g), "a2": torch.randn(H * D, r, generator=g),
         "g1": torch.randn(r, W, generator=g), "g2": torch.randn(H * V, r, generator=g), "o": torch.eye(H * V)}
    w = {k: v.double() for k, v in w.items()}
    h = 0.3 * torch.randn(T, W, generator=g).double()
    want = plain.channel_delta(h, w, "", m, 1e-5)
    # what the kernel is given: the rows after convolution and activation, and the other projections
    silu = lambda z: z * torch.sigmoid(z)
    qkv = torch.cat([silu(h @ w["q"].T), silu(h @ w["k"].T), silu(h @ w["v"].T)], dim=1).float()
    beta = (h @ w["b"].T).float()
    ag = torch.cat([(h @ w["a1"].T) @ w["a2"].T, (h @ w["g1"].T) @ w["g2"].T], dim=1).float()
    ops = TorchOps("cpu")
    state = torch.randn(3, H, V, D, generator=g)
    state[2].zero_()
    out = torch.empty(T, H * V)
    at = 0
    for n in (4, 1, 1, 2, 11):
        step = _Step([n], [2])
        ops.delta_rule(qkv[at:at + n], beta[at:at + n], ag[at:at + n], w["A_log"].float(), w["dt_bias"].float(),
                       w["norm"].float(), 1e-5, state, step, out[at:at + n], H, G, D, V)
        at += n
    torch.testing.assert_close(out.double(), want, atol=2e-5, rtol=1e-4)


def test_attention_stand_in_has_window_kept_keys_cap_and_sink():
    """One layer's attention through the stand-in's q/k preparation and attention, against the plain function."""
    import types
    g = torch.Generator().manual_seed(9)
    T, W, H, G, D, P = 45, 20, 4, 2, 8, 16
    m = {"heads": H, "kv_heads": G, "dim": D, "scale": 0.7, "softcap": 3.0, "mask": {"size": 11, "keep_first": 5},
         "rot": {"base": 100.0, "dims": 4}}
    w = {"q": torch.randn(H * D, W, generator=g), "q.b": torch.randn(H * D, generator=g),
         "k": torch.randn(G * D, W, generator=g), "k.b": torch.randn(G * D, generator=g),
         "temp": 1 + 0.3 * torch.rand(H, generator=g), "o": torch.eye(H * D), "o.b": torch.zeros(H * D)}
    w = {k: v.double() for k, v in w.items()}
    h = torch.randn(T, W, generator=g).double()
    want = plain.window_sink_attention(h, w, "", m)
    ops = TorchOps("cpu")
    qk = torch.cat([h @ w["q"].T, h @ w["k"].T], dim=1).float()
    half = 2
    ang = torch.outer(torch.arange(T).double(), 100.0 ** (-torch.arange(half).double() / half))
    pages = [2, 0, 3]
    kp, vp = torch.zeros(4, G, P, D), torch.zeros(4, G, P, D)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32)
    out, at = torch.empty(T, H, D), 0
    for n in (7, 1, 20, 1, 16):
        pos = torch.arange(at, at + n)
        slots = i32([pages[p // P] * P + p % P for p in pos.tolist()])
        grp = types.SimpleNamespace(page_table=i32(pages), cu_pages=i32([0, 3]), kv_start=i32([0]))
        step = types.SimpleNamespace(groups=[grp], n_seqs=1, cu_q=i32([0, n]), q_start=i32([at]))
        q = torch.empty(n, H, D)
        ops.qk_prepare(qk[at:at + n], H, G, D, torch.cat([w["q.b"], w["k.b"]]).float(), pos.int(), ang.cos().float(),
                       ang.sin().float(), 4, q, kp, vp, slots)
        ops.attention(q, out[at:at + n], kp, vp, step, 0, 0.7, 11, head_scale=w["temp"].float(), softcap=3.0,
                      keep_first=5, sink=True)
        at += n
    torch.testing.assert_close(out.reshape(T, H * D).double(), want, atol=2e-5, rtol=1e-4)


def test_token_input_and_squared_relu_stand_ins():
    g = torch.Generator().manual_seed(2)
    T, W, S, L = 6, 12, 3, 4
    w = {"side.embed": torch.randn(30, L * S, generator=g), "l2.side.gate": torch.randn(S, W, generator=g),
         "l2.side.proj": torch.randn(W, S, generator=g), "l2.side.norm": torch.rand(W, generator=g)}
    w = {k: v.double() for k, v in w.items()}
    x = torch.randn(T, W, generator=g)
    d = torch.randn(T, W, generator=g)
    toks = torch.randint(0, 30, (T,), generator=g)
    want = (x + d).double() + plain.token_side((x + d).double(), toks, w, 2, S, 1e-5)
    h = x.clone()
    TorchOps("cpu").token_side(h, d, toks.int(), w["side.embed"].float(), 2 * S, w["l2.side.gate"].float(),
                               w["l2.side.proj"].float(), w["l2.side.norm"].float(), 1e-5)
    torch.testing.assert_close(h.double(), want, atol=1e-4, rtol=1e-4)       # 32-bit sums against 64-bit ones
    a = torch.randn(5, 7, generator=g)
    torch.testing.assert_close(TorchOps("cpu").relu_sq(a.clone()), torch.relu(a) ** 2)


# ------------------------------------------------------------------ the engine's host side against the plain model
LENGTHS = {"a": 5, "b": 17, "c": 33, "d": 100, "e": 64, "f": 131, "g": 1, "h": 47}


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
            torch.testing.assert_close(got[(rid, p)], want[p], atol=3e-4, rtol=1e-4,
                                       msg=lambda m: f"request {rid} position {p} (first wrong place): {m}")
    assert not runner.cache.live and all(g.pages.in_use() == 0 for g in runner.cache.groups)


def test_a_freed_slot_starts_from_zero_again(tmp_path_factory):
    """A request that takes over the slot and pages of a longer one must not see what that one left."""
    folder = make_folder(tmp_path_factory, "b")
    cfg, w = plain.read_folder(folder)
    runner = runner_for(folder, 128, max_live=1)
    first = tt.random_tokens(cfg["vocab"], 90, seed=1)
    second = tt.random_tokens(cfg["vocab"], 30, seed=2)
    tt.run_in_process(runner, tt.whole({"x": first}))
    got = tt.run_in_process(runner, tt.portions({"y": second}, sizes=(2, 3, 1, 9)))
    want = plain.logits(cfg, w, second)
    for p in range(len(second)):
        torch.testing.assert_close(got[("y", p)], want[p], atol=3e-4, rtol=1e-4)
