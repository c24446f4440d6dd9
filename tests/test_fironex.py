"""Fironex through the engine against the slow oracle (tests/fironex_oracle):
each mixer alone, whole prompts against portions and single-token decoding,
mixed batches, reuse of cache pages and state slots, keys far back, at page
borders and at the edges of the sliding window, the first tokens, long
decoding, odd sizes, and greedy generation through add_request/step. Runs on
CPU; the same cases run on the HIP kernels under the gpu marker."""
import copy
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(__file__))
import fironex_oracle as oracle  # noqa: E402
import fironex_util as U  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
FULL = [U.ATTN, U.LATENT, U.RGLRU, U.latent_from(1), U.ATTN_FULL,
        U.RGLRU_WIDE]


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


def _check(eng, cfg, W, toks, plans, tol=U.TOL["float32"], want=None):
    want = oracle.forward(cfg, W, toks) if want is None else want
    for k, sizes in enumerate(plans):
        got = U.replay(eng, f"r{k}", toks, sizes)
        assert U.rel_err(got, want) < tol, sizes
    return want


# -- each mechanism alone ------------------------------------------------------
LAYERS_ALONE = {
    "attention": [U.ATTN], "attention_full": [U.ATTN_FULL],
    "latent": [U.LATENT], "latent_shared": [U.LATENT, U.latent_from(0)],
    "rglru": [U.RGLRU], "rglru_wide": [U.RGLRU_WIDE]}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(LAYERS_ALONE))
def test_single_mixer(tmp_path, device, name):
    path, cfg, W = _case(tmp_path, LAYERS_ALONE[name], seed=3)
    toks = U.tokens_for(cfg, 45, 0)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[45], [1]])


def test_residual_stream_after_every_layer(full_ckpt):
    """The model's layer taps against the oracle's, layer by layer."""
    from dynamo_amd.engine.scheduler import ScheduledSeq, SchedulerOutput
    path, cfg, W = full_ckpt
    toks = U.tokens_for(cfg, 30, 1)
    want = []
    oracle.forward(cfg, W, toks, want)
    eng = U.make_engine(path, "cpu")
    # one prefill step by hand so that the tap list can be passed
    eng.replay_step([("t", [], [])])
    req = eng.requests["t"]
    req.prompt_tokens.extend(toks)
    req.kv.ensure_capacity(len(toks))
    sched = SchedulerOutput()
    sched.prefills.append(ScheduledSeq(req, len(toks), False))
    ids, meta = eng.runner.prepare(sched)
    got = []
    with torch.inference_mode():
        eng.runner.model.forward(ids, eng.runner.kv_pool, meta, tap=got)
    assert len(got) == len(want) == len(FULL)
    for a, b in zip(got, want):
        assert float((a.double() - b).abs().max()) < 2e-4 * float(b.abs().max())


def test_ops_carry_state_across_portions():
    """Op level, CPU: the gated linear scan and the convolution continued
    over three portions from a dirty slot equal one pass."""
    from dynamo_amd.ops import seq as sops
    torch.manual_seed(0)
    T, C, nb, taps = 13, 12, 3, 4
    bw = C // nb
    x = torch.randn(T, 2 * C)
    cw, cb = torch.randn(C, taps), torch.randn(C)
    wg = torch.randn(nb, bw, 2 * bw)
    br, bi, lam = torch.randn(C), torch.randn(C), torch.randn(C) - 2

    def run(cuts):
        S = torch.full((3, C), 5.0)                      # dirty slots
        cs = torch.full((3, taps - 1, C), -3.0)
        outs, pos = [], 0
        for n in cuts:
            sb = sops.SeqBatch(torch.zeros(n, dtype=torch.int32),
                               *(torch.tensor([v], dtype=torch.int32)
                                 for v in (0, n, 1, pos)),
                               host=[(0, n, 1, pos)])
            xs = x[pos:pos + n]
            u = sops.causal_conv(xs, C, cw, cb, False, cs, sb)
            g = torch.bmm(u.view(n, nb, bw).transpose(0, 1), wg)
            outs.append(sops.rglru_scan(u, g, br, bi, lam, xs[:, C:], S, sb,
                                        8.0, torch.float32))
            pos += n
        return torch.cat(outs)
    assert torch.allclose(run([13]), run([2, 1, 10]), atol=1e-5)
    assert torch.allclose(run([13]), run([1] * 13), atol=1e-5)


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
    """145 single-token steps: the window passes over decoded tokens, pages
    fill and the recurrent state is carried step by step."""
    path, cfg, W = full_ckpt
    toks = U.tokens_for(cfg, 150, 3)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[5, 1]])


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


# -- far keys, page borders, window edges --------------------------------------
def _sharpen_latent(W, layer=0, by=5.0):
    W[f"l{layer}.mix.q"].mul_(by)
    W[f"l{layer}.mix.uk"].mul_(by / 2)


@pytest.mark.parametrize("device", DEVICES)
def test_sharp_latent_attention_far_keys_and_page_edges(tmp_path, device):
    """Queries and keys scaled up so that the softmax picks single keys,
    often hundreds of tokens back. A key read from a wrong page slot, or a
    second latent layer reading another cache than the first one's, shows."""
    def edit(W):
        _sharpen_latent(W, 0)
        _sharpen_latent(W, 1)
    path, cfg, W = _case(tmp_path, [U.LATENT, U.latent_from(0, mlp=False)],
                         seed=7, edit=edit)
    toks = U.tokens_for(cfg, 300, 4)
    eng = U.make_engine(path, device, pages=20, page_size=16)
    _check(eng, cfg, W, toks, [[15, 1, 1, 1, 32, 200, 1]])
    # and a second request over the same, now used, pages
    _check(eng, cfg, W, toks[::-1], [[17, 2]])


def test_sharp_latent_attention_really_looks_far():
    """The construction above is only a test if far keys do win."""
    cfg = U.make_config([U.LATENT])
    W = U.random_weights(cfg, 7)
    _sharpen_latent(W, 0)
    toks = U.tokens_for(cfg, 300, 4)
    m = cfg["layers"][0]["mixer"]
    h = oracle.layer_norm(oracle.d(W["embed"])[toks], W["l0.norm1"], 1e-5)
    c, kr = oracle.latent_kv(h, W, "l0.mix.", m, 1e-5)
    q = (h @ oracle.d(W["l0.mix.q"]).t()).view(300, m["heads"], -1)
    kn = (c @ oracle.d(W["l0.mix.uk"]).t()).view(300, m["heads"], m["dim"])
    far = 0.0
    for t in (299, 250, 200):
        s = (kn[:t + 1, 0] @ q[t, 0, :m["dim"]]) * m["scale"]
        far = max(far, float(torch.softmax(s, 0)[:t - 100].sum()))
    assert far > 0.2


def _window_case(W_size, i, j, dk=8, dv=6, ps=4, strong=40.0, seed=0):  # noqa
    """One kv head, two maps, T = i + 1 tokens. Map 0's key j points along
    query i with a large norm, so it takes all the weight if visible; map 1
    likewise for key j + 1. Returns q, k, v as [T, ...] tensors."""
    g = torch.Generator().manual_seed(seed)
    T = i + 1
    q = torch.randn(T, 1, 2, dk, generator=g)
    k = torch.randn(T, 1, 2, dk, generator=g) * 0.3
    v = torch.randn(T, 1, dv, generator=g)
    k[j, 0, 0] = strong * q[i, 0, 0] / q[i, 0, 0].norm()
    if j + 1 < T:
        k[j + 1, 0, 1] = strong * q[i, 0, 1] / q[i, 0, 1].norm()
    return q, k, v


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("window,ps", [(5, 4), (16, 16), (64, 16), (70, 64),
                                       (1, 4)])
@pytest.mark.parametrize("decode", [False, True], ids=["prompt", "decoded"])
def test_window_edges_at_op_level(device, window, ps, decode):
    """A dominating key placed just outside, then just inside the window of
    the last row (and its neighbour in the other key map): an edge that is
    one token off moves the whole output. Rows run as one prompt portion,
    or the last row as a decoded token over a cache filled before."""
    from dynamo_amd.ops import seq as sops
    i = 2 * window + 37
    for j in (i - window, i - window + 1):
        q, k, v = _window_case(window, i, j, ps=ps, seed=window + j)
        T, dk, dv = i + 1, q.shape[-1], v.shape[-1]
        npg = -(-T // ps)
        perm = torch.randperm(npg + 3)[:npg]              # scattered pages
        kc = torch.zeros(npg + 3, 1, ps, 2 * dk)
        vc = torch.zeros(npg + 3, 1, ps, dv)
        for t in range(T):
            kc[perm[t // ps], 0, t % ps] = k[t, 0].reshape(-1)
            vc[perm[t // ps], 0, t % ps] = v[t, 0]
        rows = [i] if decode else list(range(T))
        n = len(rows)
        sb = sops.SeqBatch(
            torch.zeros(n, dtype=torch.int32),
            *(torch.tensor([x], dtype=torch.int32) for x in (0, n, 0, rows[0])),
            page_table=perm.to(torch.int32).view(1, -1), host=[(0, n, 0, rows[0])],
            num_decode=1 if decode else 0)
        pos = torch.tensor(rows, dtype=torch.int32)
        qq = q[rows].reshape(n, -1).contiguous()
        dev = torch.device(device)
        if dev.type == "cuda":
            sb = sops.SeqBatch(sb.tok_seq.to(dev), sb.seq_start.to(dev),
                               sb.seq_len.to(dev), sb.seq_slot.to(dev),
                               sb.seq_pos0.to(dev), sb.page_table.to(dev),
                               num_decode=sb.num_decode)
        got = sops.paged_attention_rows(
            qq.to(dev), 0, 1, 2, kc.to(dev), vc.to(dev), dv, pos.to(dev), sb,
            0.5, window).cpu()
        for m in range(2):
            want = oracle.masked_softmax_attention(
                q[:, 0, m].double(), k[:, 0, m].double(), v[:, 0].double(),
                0.5, window)
            assert torch.allclose(got[-1, 0, m].double(), want[i], atol=2e-4), \
                (j - (i - window), m)
        # the dominating key decides: outside -> ignored, inside -> taken
        inside = j > i - window
        hit = torch.allclose(got[-1, 0, 0], v[j, 0], atol=1e-3)
        assert hit == inside


@pytest.mark.parametrize("device", DEVICES)
def test_sharp_window_attention_through_engine(tmp_path, device):
    """Sharp differential attention under a small window over a long
    prompt and long decoding: the strongest visible key often lies at the
    window's far edge or at a page border; both maps matter because
    lambda is made large."""
    def edit(W):
        W["l0.mix.q"].mul_(5.0)
        W["l0.mix.k"].mul_(5.0)
        W["l0.mix.lq1"].fill_(0.25)
        W["l0.mix.lk1"].fill_(0.25)
    layer = copy.deepcopy(U.ATTN)
    layer["mixer"]["mask"]["size"] = 17          # crosses 16-token pages
    path, cfg, W = _case(tmp_path, [layer], seed=9, edit=edit)
    toks = U.tokens_for(cfg, 140, 5)
    eng = U.make_engine(path, device, pages=20, page_size=16)
    _check(eng, cfg, W, toks, [[140], [40, 1], [16, 17, 1, 15, 2, 1]])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("size", [1, 2, 16, 200])
def test_window_sizes(tmp_path, device, size):
    """A window of one token (each sees only itself), one that equals the
    page size, and one longer than the prompt."""
    layer = copy.deepcopy(U.ATTN)
    layer["mixer"]["mask"]["size"] = size
    path, cfg, W = _case(tmp_path, [layer], seed=11)
    toks = U.tokens_for(cfg, 50, 6)
    eng = U.make_engine(path, device, page_size=16)
    _check(eng, cfg, W, toks, [[50], [7, 9, 1]])


def test_rotary_scaling_regimes():
    """The product's frequency table against the oracle's, with all three
    regimes (kept, blended, slowed) present."""
    from dynamo_amd.models.mixers import rotary_frequencies
    rot = U.ROT_SCALED
    plain = oracle.rope_freqs({"base": rot["base"], "dims": rot["dims"]})
    want = oracle.rope_freqs(rot)
    ratio = (want / plain).tolist()
    assert any(r == 1.0 for r in ratio) and any(
        abs(r - 1 / rot["scaling"]["factor"]) < 1e-12 for r in ratio)
    assert any(1 / rot["scaling"]["factor"] + 1e-6 < r < 1 - 1e-6 for r in ratio)
    got = rotary_frequencies(rot).double().sum(0)      # hi + lo pairs
    assert torch.allclose(got, want, rtol=1e-12)


@pytest.mark.parametrize("device", DEVICES)
def test_far_positions_rotate_exactly(tmp_path, device):
    """Positions in the thousands: angles must be formed in fp32 from the
    position, not accumulated. Only the last tokens are compared."""
    path, cfg, W = _case(tmp_path, [U.ATTN, U.LATENT], seed=13, width=64)
    toks = U.tokens_for(cfg, 1500, 7)
    want = oracle.forward(cfg, W, toks)
    eng = U.make_engine(path, device, pages=30, page_size=64)
    got = U.replay(eng, "r", toks, [1490, 1])
    assert U.rel_err(got[-12:], want[-12:]) < U.TOL["float32"]


# -- recurrence -------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 6])
def test_convolution_widths(tmp_path, device, taps):
    layer = copy.deepcopy(U.RGLRU)
    layer["mixer"]["conv"] = taps
    path, cfg, W = _case(tmp_path, [layer], seed=15)
    toks = U.tokens_for(cfg, 24, 8)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[24], [1], [2, 3, 1, 1, 9, 2]])


@pytest.mark.parametrize("device", DEVICES)
def test_slow_decay_keeps_old_tokens(tmp_path, device):
    """lam very negative makes a close to 1: the state then remembers
    tokens hundreds back and sqrt(1 - a^2) is tiny; a state lost between
    steps or a cancelled 1 - a^2 shows."""
    def edit(W):
        W["l0.mix.lam"].fill_(-9.0)
    path, cfg, W = _case(tmp_path, [U.RGLRU], seed=17, edit=edit)
    toks = U.tokens_for(cfg, 260, 9)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[260], [200, 1], [3, 64, 1, 1, 100, 2]])


# -- sizes ----------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_odd_sizes(tmp_path, device):
    """Sizes that fit no vector width (the scalar paths of the kernels),
    three query heads per kv head, one head, a single gate block, value
    and latent sizes that are not multiples of the wave, mult = 1."""
    at = copy.deepcopy(U.ATTN)
    at["mixer"].update(heads=3, kv_heads=1, dim=10, vdim=7,
                       rot={"base": 100.0, "dims": 6}, mask={"size": 9})
    la = copy.deepcopy(U.LATENT)
    la["mixer"].update(heads=1, dim=9, rot_dim=6, vdim=11, kv_rank=13,
                       rot={"base": 77.0, "dims": 6})
    lb = U.latent_from(1, heads=5, dim=3, vdim=2)
    lb["mixer"].update(rot_dim=6, kv_rank=13, rot={"base": 77.0, "dims": 6})
    rg = copy.deepcopy(U.RGLRU)
    rg["mixer"].update(width=35, blocks=5, conv=2)
    path, cfg, W = _case(tmp_path, [at, la, lb, rg], seed=19, width=66,
                         vocab=91, mult=1.0, eps=1e-3)
    toks = U.tokens_for(cfg, 40, 10)
    eng = U.make_engine(path, device, page_size=8, pages=12)
    want = _check(eng, cfg, W, toks, [[40], [3, 1, 1, 19, 2]])
    if device != "cpu":
        e16 = U.make_engine(path, device, dtype="bfloat16", page_size=8,
                            pages=12)
        _check(e16, cfg, W, toks, [[40], [3, 1, 1, 19, 2]],
               tol=U.TOL["bfloat16"], want=want)


@pytest.mark.parametrize("device", DEVICES)
def test_large_heads(tmp_path, device):
    """Head sizes of real models: 128-wide maps, a 256 + 64 latent row and
    eight query heads per kv head (the vector paths of the kernels)."""
    at = copy.deepcopy(U.ATTN)
    at["mixer"].update(heads=8, kv_heads=1, dim=128, vdim=128, scale=0.09,
                       rot={"base": 10000.0, "dims": 128}, mask={"size": 33})
    la = copy.deepcopy(U.LATENT)
    la["mixer"].update(heads=8, dim=64, rot_dim=64, vdim=64, kv_rank=256,
                       scale=0.09, rot={"base": 10000.0, "dims": 64})
    path, cfg, W = _case(tmp_path, [at, la], seed=21, width=128)
    toks = U.tokens_for(cfg, 90, 11)
    eng = U.make_engine(path, device, page_size=16, pages=12)
    _check(eng, cfg, W, toks, [[90], [70, 1]])


@pytest.mark.parametrize("device", DEVICES)
def test_wide_latent_partly_rotated(tmp_path, device):
    """A latent wider than 512 (the widest value row of the matrix-core
    kernel) whose rotated part is only half rotated."""
    la = copy.deepcopy(U.LATENT)
    la["mixer"].update(heads=2, dim=8, rot_dim=16, vdim=8, kv_rank=600,
                       rot={"base": 300.0, "dims": 8})
    lb = U.latent_from(0, heads=3, dim=8, vdim=16, mlp=False)
    lb["mixer"].update(rot_dim=16, kv_rank=600, rot={"base": 300.0, "dims": 8})
    path, cfg, W = _case(tmp_path, [la, lb], seed=23, width=48, vocab=61)
    toks = U.tokens_for(cfg, 70, 12)
    eng = U.make_engine(path, device, page_size=16, pages=8)
    want = _check(eng, cfg, W, toks, [[70], [50, 1]])
    if device != "cpu":
        e16 = U.make_engine(path, device, dtype="bfloat16", page_size=16, pages=8)
        _check(e16, cfg, W, toks, [[33, 2, 1]], tol=U.TOL["bfloat16"], want=want)


def test_bad_configs_are_refused(tmp_path):
    from dynamo_amd.models.registry import build_model, resolve_model_config
    later = U.make_config([U.latent_from(1), U.LATENT])
    other = U.make_config([U.LATENT, U.latent_from(0)])
    other["layers"][1]["mixer"]["kv_rank"] = 24
    for k, cfg in enumerate((later, other)):
        d = tmp_path / str(k)
        os.makedirs(d)
        import json
        with open(d / "config.json", "w") as f:
            json.dump(cfg, f)
        with pytest.raises(ValueError):
            build_model(resolve_model_config(str(d)), "cpu", torch.float32)


def test_unused_checkpoint_tensor_is_an_error(tmp_path):
    cfg = U.make_config([U.RGLRU])
    W = U.random_weights(cfg, 0)
    W["l0.mix.extra"] = torch.zeros(3, dtype=torch.bfloat16)
    path = U.write_checkpoint(tmp_path, cfg, W)
    with pytest.raises(ValueError):
        U.make_engine(path, "cpu")


# -- bf16 prompt portions on the matrix cores ---------------------------------
def _paged(k, v, ps, extra=3, seed=0):
    """Scatter [T, G, d] keys (and values) over pages in a random order."""
    T, G = k.shape[0], k.shape[1]
    npg = -(-T // ps)
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(npg + extra, generator=g)[:npg]
    kc = torch.zeros(npg + extra, G, ps, k.shape[2], dtype=k.dtype)
    vc = None if v is None else torch.zeros(npg + extra, G, ps, v.shape[2],
                                            dtype=v.dtype)
    for t in range(T):
        kc[perm[t // ps], :, t % ps] = k[t]
        if v is not None:
            vc[perm[t // ps], :, t % ps] = v[t]
    return kc, vc, perm.to(torch.int32)


def _prompt_batch(spans, tables, dev, tiled):
    """SeqBatch of prompt portions [(rows, first position)], one per page
    table row, with or without 64-row tiles."""
    from dynamo_amd.ops import seq as sops
    tok_seq, start, host, t0, tn = [], 0, [], [], []
    for si, (n, pos0) in enumerate(spans):
        host.append((start, n, si, pos0))
        tok_seq += [si] * n
        for q0 in range(0, n, 64):
            t0.append(start + q0)
            tn.append(min(64, n - q0))
        start += n
    maxp = max(len(t) for t in tables)
    pt = torch.zeros(len(tables), maxp, dtype=torch.int32)
    for i, t in enumerate(tables):
        pt[i, :len(t)] = t
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)  # noqa: E731
    cols = list(zip(*host))
    pos = torch.cat([torch.arange(p0, p0 + n) for n, p0 in spans]).to(
        torch.int32).to(dev)
    sb = sops.SeqBatch(i32(tok_seq), i32(cols[0]), i32(cols[1]), i32(cols[2]),
                       i32(cols[3]), page_table=pt.to(dev), num_decode=0,
                       tiles=(i32(t0), i32(tn)) if tiled else None)
    return sb, pos


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,dk,dv,kmaps,window,alias", [
    (4, 2, 64, 128, 2, 100, False),     # differential heads under a window
    (6, 3, 24, 40, 2, 19, False),       # sizes padded inside the kernel
    (2, 1, 128, 64, 1, 0, False),       # plain grouped attention
    (3, 1, 192, 128, 1, 0, True),       # latent rows: values alias keys
    (2, 1, 320, 256, 1, 0, True),
    (4, 1, 576, 512, 1, 0, True),
    (2, 2, 16, 8, 2, 1, False),         # a window of one token
])
def test_mfma_prompt_attention_matches_row_kernel(H, G, dk, dv, kmaps, window,
                                                  alias):
    """bf16 prompt portions (two sequences, one continued from position 70
    so that tiles start inside a page and inside the window) through the
    matrix-core kernel against the fp32-accumulating row kernel and the
    oracle."""
    from dynamo_amd.ops import seq as sops
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(dk + dv)
    ps = 16
    lens = [(130, 0), (75, 70)]          # (rows this step, first position)
    krow = kmaps * dk
    ks, vs, tabs, qs = [], [], [], []
    for n, p0 in lens:
        T = n + p0
        k = (torch.randn(T, G, krow, generator=g) * 0.7).to(torch.bfloat16)
        v = None if alias else torch.randn(T, G, dv, generator=g).to(torch.bfloat16)
        ks.append(k)
        vs.append(v)
        qs.append((torch.randn(n, H * krow, generator=g) * 0.7).to(torch.bfloat16))
    # one cache for both sequences: pages of the second follow the first's
    kc0, vc0, t0 = _paged(ks[0], vs[0], ps, seed=1)
    kc1, vc1, t1 = _paged(ks[1], vs[1], ps, seed=2)
    kc = torch.cat([kc0, kc1])
    vc = None if alias else torch.cat([vc0, vc1])
    tabs = [t0, t1 + kc0.shape[0]]
    q = torch.cat(qs)
    outs = []
    for tiled in (False, True):
        sb, pos = _prompt_batch(lens, tabs, dev, tiled)
        outs.append(sops.paged_attention_rows(
            q.to(dev), 0, H, kmaps, kc.to(dev), None if alias else vc.to(dev),
            dv, pos, sb, 0.11, window).cpu())
    assert torch.isfinite(outs[1]).all()
    scale = float(outs[0].abs().max())
    assert float((outs[0] - outs[1]).abs().max()) < 2e-3 * scale
    # the oracle on the same bf16 inputs, last rows of each sequence
    row = 0
    for (n, p0), k, v, qq in zip(lens, ks, vs, qs):
        T = n + p0
        kd = k.double().view(T, G, kmaps, dk)
        vd = kd.reshape(T, G, krow)[:, :, :dv] if alias else v.double()
        for h in (0, H - 1):
            for mp in range(kmaps):
                qfull = torch.zeros(T, dk, dtype=torch.float64)
                qfull[p0:] = qq.double().view(n, H, kmaps, dk)[:, h, mp]
                want = oracle.masked_softmax_attention(
                    qfull, kd[:, h // (H // G), mp], vd[:, h // (H // G)],
                    0.11, window or None)[p0:]
                got = outs[1][row:row + n, h, mp].double()
                assert float((got - want).abs().max()) < 2e-3 * scale, (h, mp)
        row += n


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,dk,dv,kmaps,window,alias", [
    (16, 1, 576, 512, 1, 0, True),      # latent rows, 16 heads on one row
    (5, 1, 192, 128, 1, 0, True),       # fewer heads than a tile has rows
    (80, 1, 64, 64, 1, 0, False),       # more heads than one tile (64 + 16)
    (16, 2, 64, 128, 2, 100, False),    # differential heads, 8 per kv head
])
def test_mfma_decode_matches_row_kernel(H, G, dk, dv, kmaps, window, alias):
    """Single decoded tokens of sequences of unequal length (one of them a
    padding row, one a sequence of one token) with heads as tile rows and
    the keys split over workgroups, against the row kernel."""
    from dynamo_amd.ops import seq as sops
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(H + dk)
    ps, krow = 16, kmaps * dk
    ctx = [700, 1, 64, 65, 333, 129]
    pad = 2                                  # this row's seq_len is 0
    caches, tabs, base = [], [], 0
    for n in ctx:
        k = (torch.randn(n, G, krow, generator=g) * 0.6).to(torch.bfloat16)
        v = None if alias else torch.randn(n, G, dv, generator=g).to(torch.bfloat16)
        kc, vc, tab = _paged(k, v, ps, extra=1, seed=n)
        caches.append((kc, vc))
        tabs.append(tab + base)
        base += kc.shape[0]
    kc = torch.cat([c[0] for c in caches]).to(dev)
    vc = None if alias else torch.cat([c[1] for c in caches]).to(dev)
    B = len(ctx)
    pt = torch.zeros(B, max(len(t) for t in tabs), dtype=torch.int32)
    for i, t in enumerate(tabs):
        pt[i, :len(t)] = t
    q = (torch.randn(B, H * krow, generator=g) * 0.6).to(torch.bfloat16).to(dev)
    rows = torch.arange(B, dtype=torch.int32, device=dev)
    lens = torch.ones(B, dtype=torch.int32)
    lens[pad] = 0
    pos = torch.tensor([n - 1 for n in ctx], dtype=torch.int32, device=dev)
    outs = []
    for ndec in (0, B):                      # row kernel, then matrix cores
        sb = sops.SeqBatch(rows, rows, lens.to(dev), rows, pos,
                           page_table=pt.to(dev), num_decode=ndec)
        o = sops.paged_attention_rows(q, 0, H, kmaps, kc, vc, dv, pos, sb,
                                      0.09, window).cpu()
        outs.append(torch.cat([o[:pad], o[pad + 1:]]))
    assert torch.isfinite(outs[1]).all()
    scale = float(outs[0].abs().max())
    assert float((outs[0] - outs[1]).abs().max()) < 2e-3 * scale


@pytest.mark.gpu
@pytest.mark.parametrize("window", [5, 64, 70])
def test_window_edges_on_the_matrix_cores(window):
    """The dominating key just outside / just inside the window, bf16
    prompt tiles: the last row of the last tile decides."""
    from dynamo_amd.ops import seq as sops
    dev = torch.device("cuda:0")
    i = 2 * window + 37
    for j in (i - window, i - window + 1):
        q, k, v = _window_case(window, i, j, dk=16, dv=8, seed=window + j)
        q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
        T = i + 1
        kc, vc, tab = _paged(k.reshape(T, 1, -1), v, 16, seed=3)
        sb, pos = _prompt_batch([(T, 0)], [tab], dev, True)
        got = sops.paged_attention_rows(
            q.reshape(T, -1).to(dev), 0, 1, 2, kc.to(dev), vc.to(dev), 8, pos,
            sb, 0.5, window).cpu()
        inside = j > i - window
        hit = torch.allclose(got[-1, 0, 0], v[j, 0].float(), atol=2e-2)
        assert hit == inside
        want = oracle.masked_softmax_attention(
            q[:, 0, 1].double(), k[:, 0, 1].double(), v[:, 0].double(), 0.5,
            window)
        assert torch.allclose(got[:, 0, 1].double(), want, atol=2e-2)


# -- bf16 and graphs ---------------------------------------------------------
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


MANY_HEADS = [
    {"type": "latent_attention",
     "mixer": {"heads": 8, "dim": 32, "rot_dim": 16, "vdim": 24, "kv_rank": 64,
               "scale": 0.15, "rot": {"base": 5000.0, "dims": 16}},
     "mlp": {"kind": "dense", "ff": 144}},
    {"type": "attention",
     "mixer": {"heads": 16, "kv_heads": 2, "dim": 16, "vdim": 24,
               "scale": 0.25, "diff": 0.4, "mask": {"size": 37},
               "rot": U.ROT_SCALED},
     "mlp": None},
    U.RGLRU,
    {"type": "latent_attention",
     "mixer": {"heads": 12, "dim": 16, "rot_dim": 16, "vdim": 8, "kv_rank": 64,
               "scale": 0.2, "kv_from": 0,
               "rot": {"base": 5000.0, "dims": 16}},
     "mlp": {"kind": "dense", "ff": 120}},
]


@pytest.mark.gpu
def test_bf16_many_heads_mixed_batches_and_graphs(tmp_path):
    """Head groups of 8 and more in bf16: prompt tiles and decoded tokens
    both run on the matrix cores, side by side in mixed batches over a
    small pool, and in captured decode graphs."""
    from dynamo_amd.engine import SamplingParams
    path, cfg, W = _case(tmp_path, MANY_HEADS, seed=31, width=128)
    lens = {"a": 150, "b": 9, "c": 77, "d": 1, "e": 66}
    toks = {k: U.tokens_for(cfg, n, 70 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: oracle.forward(cfg, W, t) for k, t in toks.items()}
    eng = U.make_engine(path, "cuda:0", dtype="bfloat16", pages=22, slots=3,
                        page_size=16)
    plan = [[("a", 70), ("b", 5), ("d", 1)],
            [("a", 1), ("b", 1)],
            [("a", 1), ("b", 1), ("c", 64)],
            [("a", 66), ("b", 2), ("c", 1)],
            [("a", 1), ("c", 12), ("e", 65)],
            [("a", 1), ("e", 1)],
            [("a", 10)]]
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
        assert U.rel_err(torch.cat(got[rid]), want[rid]) < U.TOL["bfloat16"], rid
    # greedy decoding through captured graphs stays on the oracle's best
    # tokens (up to bf16 noise in near ties)
    e = U.make_engine(path, "cuda:0", dtype="bfloat16", graphs=True, slots=4,
                      pages=40, page_size=16)
    prompts = {f"g{i}": U.tokens_for(cfg, 30 + 17 * i, 90 + i) for i in range(3)}
    for rid, p in prompts.items():
        e.add_request(rid, p, SamplingParams(max_tokens=24, ignore_eos=True))
    out = {k: [] for k in prompts}
    while e.has_work():
        for so in e.step():
            out[so.req_id].append(so.new_token)
    assert e.graph_runner is not None and e.graph_runner.graphs
    for rid, p in prompts.items():
        seq = list(p)
        for tok in out[rid]:
            lg = oracle.forward(cfg, W, seq)[-1]
            spread = float(lg.std())
            assert lg[tok] >= lg.max() - 0.15 * spread, (rid, len(seq))
            seq.append(tok)


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
    from dynamo_amd.models.registry import build_model, native_extensions
    cfg = PRESETS["tiny-fironex"]
    m = build_model(cfg, "cpu", torch.float32)
    # the second latent layer reads the first one's cache and owns none
    assert [s is not None for s in m.kv_layer_shapes()] == [True, False, False, True]
    assert [len(s) for s in m.state_layer_shapes()] == [0, 2, 0, 0]
    assert native_extensions(cfg, "cuda:0") == ["_core", "_hip_seq"]


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
