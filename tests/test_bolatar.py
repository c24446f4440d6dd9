"""Bolatar through the engine against the slow oracle (tests/bolatar_oracle):
each mixer alone, whole prompts against portions and single-token decoding,
mixed batches, reuse of cache pages and state slots, edges of pages, of the
query-temperature period and of the convolution, long decoding, and greedy
generation through add_request/step. Runs on CPU; the same cases run on the
HIP kernels under the gpu marker."""
import copy
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(__file__))
import bolatar_oracle as oracle  # noqa: E402
import bolatar_util as U  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
FULL = [U.PARALLEL, U.DELTA, U.MLSTM, U.DELTA_WIDE]


@pytest.fixture(scope="module")
def full_ckpt(tmp_path_factory):
    cfg = U.make_config(FULL)
    W = U.random_weights(cfg, 1)
    return U.write_checkpoint(tmp_path_factory.mktemp("full"), cfg, W), cfg, W


def _case(tmp_path, layers, seed=0, edit=None, **kw):
    cfg = U.make_config(layers, **kw)
    W = U.random_weights(cfg, seed)
    if edit:
        edit(W)
    return U.write_checkpoint(tmp_path, cfg, W), cfg, W


# -- each mechanism alone ------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("layer", [U.DELTA, U.DELTA_WIDE, U.PARALLEL, U.MLSTM],
                         ids=["delta", "delta_wide", "parallel", "mlstm"])
def test_single_mixer(tmp_path, device, layer):
    path, cfg, W = _case(tmp_path, [layer], seed=3)
    toks = U.tokens_for(cfg, 45, 0)
    want = oracle.forward(cfg, W, toks)
    eng = U.make_engine(path, device)
    assert U.rel_err(U.replay(eng, "a", toks, [45]), want) < U.TOL["float32"]
    assert U.rel_err(U.replay(eng, "b", toks, [1]), want) < U.TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("keep", ["left", "right"])
def test_parallel_branches_apart(tmp_path, device, keep):
    """Silence one branch of the parallel mixer so the other cannot hide."""
    drop = "right" if keep == "left" else "left"

    def edit(W):
        W[f"l0.mix.{drop}.out"].zero_()
    path, cfg, W = _case(tmp_path, [U.PARALLEL], seed=5, edit=edit)
    toks = U.tokens_for(cfg, 40, 1)
    want = oracle.forward(cfg, W, toks)
    eng = U.make_engine(path, device)
    assert U.rel_err(U.replay(eng, "a", toks, [7, 2, 1]), want) < U.TOL["float32"]


def test_mechanism_functions_agree_with_ops():
    """Op level, CPU: state carried across two portions equals one pass."""
    from dynamo_amd.ops import seq as sops
    torch.manual_seed(0)
    T, H, dk, dv = 11, 2, 8, 12
    r, k = torch.randn(T, H * dk), torch.randn(T, H * dk)
    v, wr = torch.randn(T, H * dk), torch.randn(T, H * dk)
    w0, u = torch.randn(H * dk) - 2, torch.randn(H, dk)

    def run(cuts):
        state = torch.full((3, H, dk, dk), 7.0)      # dirty slot
        outs, pos = [], 0
        for n in cuts:
            sb = sops.SeqBatch(torch.zeros(n, dtype=torch.int32),
                               *(torch.tensor([x], dtype=torch.int32)
                                 for x in (0, n, 2, pos)),
                               host=[(0, n, 2, pos)])
            outs.append(sops.rwkv_time_mix(r[pos:pos + n], k[pos:pos + n],
                                           v[pos:pos + n], wr[pos:pos + n],
                                           w0, u, state, sb, H))
            pos += n
        return torch.cat(outs)
    assert torch.allclose(run([11]), run([4, 1, 6]), atol=1e-5)


# -- portions, decoding, first tokens -----------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2], [3, 2, 2, 17, 5, 1], [31, 33, 2, 1],
                                   [64, 1]], ids=str)
def test_portions_match_whole(full_ckpt, device, sizes):
    path, cfg, W = full_ckpt
    toks = U.tokens_for(cfg, 83, 2)
    want = oracle.forward(cfg, W, toks)
    eng = U.make_engine(path, device)
    got = U.replay(eng, "r", toks, sizes)
    assert U.rel_err(got, want) < U.TOL["float32"]
    # the first tokens of a sequence, alone
    assert U.rel_err(got[:3], want[:3]) < U.TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode(full_ckpt, device):
    path, cfg, W = full_ckpt
    toks = U.tokens_for(cfg, 150, 3)
    want = oracle.forward(cfg, W, toks)
    eng = U.make_engine(path, device)
    got = U.replay(eng, "r", toks, [5, 1])      # 145 single-token steps
    assert U.rel_err(got, want) < U.TOL["float32"]


# -- batches, reuse of pages and slots ----------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_with_reuse(full_ckpt, device):
    """Unequal requests share steps (portions beside single tokens); the
    pool is so small that finished requests' pages and slots are taken
    again at once, at other places than before."""
    path, cfg, W = full_ckpt
    lens = {"a": 70, "b": 9, "c": 37, "d": 1, "e": 50, "f": 23}
    toks = {k: U.tokens_for(cfg, n, 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: oracle.forward(cfg, W, t) for k, t in toks.items()}
    eng = U.make_engine(path, device, pages=11, slots=3, page_size=16)
    plan = [  # (request, tokens this step)
        [("a", 2), ("b", 5), ("d", 1)],
        [("a", 30), ("b", 1)],
        [("a", 1), ("b", 1), ("c", 17)],
        [("b", 2), ("c", 3), ("a", 1)],
        [("a", 36), ("c", 1)],
        [("c", 16), ("e", 2)],
        [("e", 31), ("f", 23)],
        [("e", 1)], [("e", 16)],
    ]
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    for step in plan:
        entries, end = [], []
        for rid, n in step:
            entries.append((rid, toks[rid][at[rid]:at[rid] + n], list(range(n))))
            at[rid] += n
            if at[rid] == lens[rid]:
                end.append(rid)
        lg = eng.replay_step(entries, end).cpu()
        row = 0
        for rid, n in step:
            got[rid].append(lg[row:row + n])
            row += n
    assert at == lens
    for rid in lens:
        assert U.rel_err(torch.cat(got[rid]), want[rid]) < U.TOL["float32"], rid
    assert eng.alloc.num_free == 11 and eng.state_slots.num_free == 3


def test_pool_exhaustion_raises(full_ckpt):
    path, cfg, W = full_ckpt
    eng = U.make_engine(path, "cpu", pages=2, slots=1)
    eng.replay_step([("a", U.tokens_for(cfg, 20, 0), [])])
    with pytest.raises(MemoryError):
        eng.replay_step([("b", [1, 2], [])])              # no slot
    with pytest.raises(MemoryError):
        eng.replay_step([("a", U.tokens_for(cfg, 20, 1), [])])  # no page


# -- far keys, page borders, temperature period ------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_sharp_attention_far_keys_and_page_edges(tmp_path, device):
    """Queries and keys scaled up so that the softmax picks single keys,
    often hundreds of tokens back; the distance penalty is kept small so
    far keys can win. Any key read from a wrong page slot shows."""
    def edit(W):
        W["l0.mix.left.q"].mul_(6.0)
        W["l0.mix.left.k"].mul_(6.0)
        W["l0.mix.left.r1"].mul_(0.05)
        W["l0.mix.right.out"].zero_()
    path, cfg, W = _case(tmp_path, [U.PARALLEL], seed=7, edit=edit)
    toks = U.tokens_for(cfg, 300, 4)
    want = oracle.forward(cfg, W, toks)
    # how far back does the strongest key lie? (sanity of the construction)
    eng = U.make_engine(path, device, pages=20, page_size=16)
    got = U.replay(eng, "r", toks, [15, 1, 1, 1, 32, 200, 1])
    assert U.rel_err(got, want) < U.TOL["float32"]
    # and a second request over the same, now used, pages
    got = U.replay(eng, "s", toks[::-1], [17, 2])
    assert U.rel_err(got, oracle.forward(cfg, W, toks[::-1])) < U.TOL["float32"]


def test_sharp_attention_really_looks_far():
    """The construction above is only a test if far keys do win."""
    cfg = U.make_config([U.PARALLEL])
    W = U.random_weights(cfg, 7)
    W["l0.mix.left.q"].mul_(6.0)
    W["l0.mix.left.k"].mul_(6.0)
    W["l0.mix.left.r1"].mul_(0.05)
    toks = U.tokens_for(cfg, 300, 4)
    Wd = {k: v.double() for k, v in W.items()}
    x = Wd["embed"][toks] * cfg["embedding"]["scale"] + Wd["pos"][:300]
    h = oracle.rms(x, 1e-5) * Wd["l0.norm1"]
    m = cfg["layers"][0]["mixer"]["left"]
    q = (h @ Wd["l0.mix.left.q"].T).view(300, m["heads"], m["dim"])
    k = (h @ Wd["l0.mix.left.k"].T).view(300, m["kv_heads"], m["dim"])
    s = torch.einsum("d,jd->j", q[299, 0], k[:, 0]) * m["scale"]
    p = torch.softmax(s, 0)
    assert p.max() > 0.5 and p[:200].sum() > 0.05


@pytest.mark.parametrize("device", DEVICES)
def test_temperature_period_edges(tmp_path, device):
    """Positions just before and at multiples of the period, in a prompt
    portion and decoded one by one, with a large coefficient."""
    layer = copy.deepcopy(U.PARALLEL)
    layer["mixer"]["left"]["q_temp"] = {"coef": 2.0, "every": 7}
    path, cfg, W = _case(tmp_path, [layer], seed=9)
    toks = U.tokens_for(cfg, 30, 5)
    want = oracle.forward(cfg, W, toks)
    eng = U.make_engine(path, device)
    for sizes in ([30], [5, 1], [6, 8, 1]):
        assert U.rel_err(U.replay(eng, "r", toks, sizes), want) < U.TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 6])
def test_convolution_widths(tmp_path, device, taps):
    layer = copy.deepcopy(U.DELTA)
    layer["mixer"]["conv"] = taps
    path, cfg, W = _case(tmp_path, [layer], seed=11)
    toks = U.tokens_for(cfg, 24, 6)
    want = oracle.forward(cfg, W, toks)
    eng = U.make_engine(path, device)
    for sizes in ([24], [1], [2, 3, 1, 1, 9, 2]):
        assert U.rel_err(U.replay(eng, "r", toks, sizes), want) < U.TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_odd_sizes(tmp_path, device):
    """Sizes that fit no vector width: the scalar paths of the kernels, a
    group of three query heads per kv head, a key size above 32 rows per
    lane group and a value size that is not a multiple of the wave."""
    par = copy.deepcopy(U.PARALLEL)
    par["mixer"]["left"].update(heads=3, kv_heads=1, dim=10, vdim=7)
    par["mixer"]["right"].update(heads=2, dim=9)
    dl = copy.deepcopy(U.DELTA)
    dl["mixer"].update(heads=2, kv_heads=1, dim=70, vdim=5)
    ml = copy.deepcopy(U.MLSTM)
    ml["mixer"].update(heads=3, dim=37, vdim=70)
    path, cfg, W = _case(tmp_path, [par, dl, ml], seed=13, width=66, vocab=91)
    toks = U.tokens_for(cfg, 40, 8)
    want = oracle.forward(cfg, W, toks)
    eng = U.make_engine(path, device, page_size=8, pages=12)
    for sizes in ([40], [3, 1, 1, 19, 2]):
        assert U.rel_err(U.replay(eng, "r", toks, sizes), want) < U.TOL["float32"]


@pytest.mark.gpu
def test_bf16_and_graph_decode(full_ckpt):
    """bf16 serving path on the GPU: logits close to the oracle, and greedy
    decoding through captured hipGraphs equals the eager engine token for
    token (every replay checked against eager work in between)."""
    from dynamo_amd.engine import SamplingParams
    path, cfg, W = full_ckpt
    toks = U.tokens_for(cfg, 70, 50)
    want = oracle.forward(cfg, W, toks)
    eng = U.make_engine(path, "cuda:0", dtype="bfloat16")
    assert U.rel_err(U.replay(eng, "r", toks, [33, 2, 1]), want) < U.TOL["bfloat16"]
    outs = []
    for graphs in (False, True):
        e = U.make_engine(path, "cuda:0", dtype="float32", graphs=graphs,
                          slots=4)
        for i in range(3):
            e.add_request(f"g{i}", U.tokens_for(cfg, 9 + 7 * i, 60 + i),
                          SamplingParams(max_tokens=20, ignore_eos=True))
        got = {}
        while e.has_work():
            for so in e.step():
                got.setdefault(so.req_id, []).append(so.new_token)
        if graphs:
            assert e.graph_runner is not None and e.graph_runner.graphs
        outs.append(got)
    assert outs[0] == outs[1]


# -- generation through the engine's own entry point ------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_matches_oracle(full_ckpt, device):
    from dynamo_amd.engine import SamplingParams
    path, cfg, W = full_ckpt
    eng = U.make_engine(path, device, pages=24, slots=2, max_batched_tokens=16)
    prompts = {"x": U.tokens_for(cfg, 21, 20), "y": U.tokens_for(cfg, 5, 21),
               "z": U.tokens_for(cfg, 40, 22)}
    for rid, p in prompts.items():     # three requests, two slots: z waits
        eng.add_request(rid, p, SamplingParams(max_tokens=12, ignore_eos=True))
    out = {k: [] for k in prompts}
    for _ in range(400):
        if not eng.has_work():
            break
        for so in eng.step():
            out[so.req_id].append(so.new_token)
    assert not eng.has_work()
    for rid, p in prompts.items():
        seq = list(p)
        for tok in out[rid]:
            lg = oracle.forward(cfg, W, seq)[-1]
            assert lg[tok] >= lg.max() - 1e-3, (rid, len(seq))
            seq.append(tok)
        assert len(out[rid]) == 12
    assert eng.state_slots.num_free == 2


def test_preempted_request_restarts_clean(full_ckpt):
    """A pool too small for two long requests: one is preempted, gives its
    slot and pages back, and recomputes from its first token."""
    from dynamo_amd.engine import SamplingParams
    path, cfg, W = full_ckpt
    eng = U.make_engine(path, "cpu", pages=6, slots=2, page_size=16,
                        max_batched_tokens=64)
    prompts = {"x": U.tokens_for(cfg, 40, 30), "y": U.tokens_for(cfg, 38, 31)}
    for rid, p in prompts.items():
        eng.add_request(rid, p, SamplingParams(max_tokens=14, ignore_eos=True))
    out = {k: [] for k in prompts}
    for _ in range(400):
        if not eng.has_work():
            break
        for so in eng.step():
            out[so.req_id].append(so.new_token)
    assert sum(r.num_preemptions for r in eng.requests.values()) >= 1
    for rid, p in prompts.items():
        seq = list(p)
        for tok in out[rid]:
            lg = oracle.forward(cfg, W, seq)[-1]
            assert lg[tok] >= lg.max() - 1e-3, (rid, len(seq))
            seq.append(tok)


def test_registry_and_preset():
    from dynamo_amd.engine.config import PRESETS
    from dynamo_amd.models.registry import build_model
    m = build_model(PRESETS["tiny-bolatar"], "cpu", torch.float32)
    assert [s is not None for s in m.kv_layer_shapes()] == [True, False, False]
    assert len(m.state_layer_shapes()[0]) == 2     # rwkv memory + last input


def test_trace_run_command(full_ckpt, tmp_path):
    import json
    import subprocess
    import numpy as np
    path, cfg, W = full_ckpt
    toks = U.tokens_for(cfg, 20, 40)
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": toks[:13], "want": [0, 12]}], "end": []},
             {"step": 1, "entries": [{"id": "q", "tokens": toks[13:14], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "q", "tokens": toks[14:], "want": [5]}], "end": ["q"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", path,
                        "--dtype", "float32", "--out", str(tmp_path / "o"),
                        "--max-tokens", "64", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == \
        ["done 0", "done 1", "done 2"]
    want = oracle.forward(cfg, W, toks)
    a = np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(2, -1)
    b = np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4").reshape(1, -1)
    assert not (tmp_path / "o" / "1.f32").exists()
    got = torch.from_numpy(np.concatenate([a, b]))
    assert U.rel_err(got, want[[0, 12, 19]]) < U.TOL["float32"]
