"""Each HIP kernel of dynamo_amd._hip_seq against the plain torch version of
the same op (ops/seq_ref.py, fp32 on the CPU), on random inputs with uneven
sizes, dirty state slots, several sequences per batch and portions that
continue earlier ones."""
import pytest
import torch

from dynamo_amd.ops import seq as sops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _batch(spans, device):
    """spans: [(len, slot, pos0)] laid out back to back."""
    host, tok, row = [], [], 0
    for i, (n, slot, pos0) in enumerate(spans):
        host.append((row, n, slot, pos0))
        tok += [i] * n
        row += n
    cols = torch.tensor(host, dtype=torch.int32).t().contiguous().to(device)
    return sops.SeqBatch(torch.tensor(tok, dtype=torch.int32, device=device),
                         cols[0], cols[1], cols[2], cols[3], host=host), row


SPANS = [(5, 2, 0), (1, 0, 9), (0, 3, 4), (12, 1, 3), (2, 4, 0)]


def _both(fn, tensors, spans=SPANS, states=()):
    """Run fn(sb, *tensors, *states) on CPU and GPU; returns outputs and the
    states after the call for both."""
    res = []
    for dev in ("cpu", DEV):
        sb, _ = _batch(spans, dev)
        st = [s.clone().to(dev) for s in states]
        out = fn(sb, *[t.clone().to(dev) for t in tensors], *st)
        res.append(([o.float().cpu() for o in
                     (out if isinstance(out, (tuple, list)) else [out])],
                    [s.cpu() for s in st]))
    return res


def _close(res, atol=2e-5, rtol=1e-4):
    (oc, sc), (og, sg) = res
    for a, b in zip(oc + sc, og + sg):
        assert torch.allclose(a, b, atol=atol, rtol=rtol), \
            float((a - b).abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rowwise_kernels(dtype):
    g = torch.Generator().manual_seed(0)
    T, W, F = 20, 150, 77
    x = torch.randn(T, W, generator=g)
    delta = torch.randn(T, W, generator=g).to(dtype)
    gain = torch.tensor([1.3])
    tol = dict(atol=2e-5) if dtype == torch.float32 else dict(atol=3e-2)

    def norm(sb, res, d, gg):
        out = sops.add_scalar_rmsnorm(res, d, gg, 1e-5, dtype)
        return out, res
    _close(_both(norm, [x, delta, gain]), **tol)

    gu = (torch.randn(T, 2 * F, generator=g) * 3).to(dtype)
    _close(_both(lambda sb, t: sops.clamped_glu(t, 2.0, 1.702), [gu]), **tol)

    a = torch.randn(T, W, generator=g).to(dtype)
    b = torch.randn(T, W, generator=g).to(dtype)
    wa, wb = torch.rand(W, generator=g) + 0.5, torch.rand(W, generator=g) + 0.5
    _close(_both(lambda sb, *t: sops.dual_rmsnorm_mean(*t, 1e-5),
                 [a, b, wa, wb]), **tol)

    o = torch.randn(T, 3, 50, generator=g)
    gate = torch.randn(T, 170, generator=g).to(dtype)
    w = torch.rand(150, generator=g) + 0.5
    for stride, act in ((0, sops.GATE_SILU), (50, sops.GATE_SIGMOID)):
        _close(_both(lambda sb, oo, ww, gg: sops.head_norm_gate(
            oo, ww, stride, gg[:, 20:], act, 1e-5, dtype), [o, w, gate]), **tol)

    emb = torch.randn(40, W, generator=g).to(dtype)
    pos = torch.randn(64, W, generator=g).to(dtype)
    ids = torch.randint(0, 40, (T,), generator=g, dtype=torch.int32)
    ps = torch.randint(0, 64, (T,), generator=g, dtype=torch.int32)
    _close(_both(lambda sb, i, p, e, q: sops.embed_scale_pos(i, p, e, q, 2.5),
                 [ids, ps, emb, pos]), atol=1e-6)

    lg = torch.randn(7, 33, generator=g) * 40
    _close(_both(lambda sb, t: sops.softcap_(t, 30.0), [lg]))


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_conv_and_shift(taps):
    g = torch.Generator().manual_seed(1)
    sb, T = _batch(SPANS, "cpu")
    C, W = 70, 90
    x = torch.randn(T, C + 13, generator=g)
    w = torch.randn(C, taps, generator=g)
    state = torch.randn(5, taps - 1, C, generator=g)
    _close(_both(lambda sb, xx, ww, st: sops.causal_conv_silu(xx, C, ww, st, sb),
                 [x, w], states=[state]))
    h = torch.randn(T, W, generator=g)
    mu = torch.rand(5, W, generator=g)
    prev = torch.randn(5, W, generator=g)
    _close(_both(lambda sb, hh, mm, st: sops.token_shift_mix(hh, mm, st, sb),
                 [h, mu], states=[prev]))


@pytest.mark.parametrize("dk,dv", [(24, 16), (70, 5), (128, 130)])
def test_recurrences(dk, dv):
    g = torch.Generator().manual_seed(2)
    sb, T = _batch(SPANS, "cpu")
    H, G = 4, 2
    qkv = torch.randn(T, 2 * G * dk + H * dv, generator=g)
    proj = torch.randn(T, 2 * H + 3, generator=g)
    A, dt = -torch.rand(H, generator=g) * 3, -torch.rand(H, generator=g)
    S = torch.randn(5, H, dk, dv, generator=g) * 0.1
    _close(_both(lambda sb, q, p, a, d, st: sops.gated_delta_rule(
        q.clone(), p, 1, 1 + H, a, d, st, sb, H, G, dv, dk ** -0.5),
        [qkv, proj, A, dt], states=[S]), atol=1e-4)

    r, k, wr = (torch.randn(T, H * dk, generator=g) for _ in range(3))
    v = torch.randn(T, H * dk, generator=g)
    w0 = torch.randn(H * dk, generator=g) - 2
    u = torch.randn(H, dk, generator=g)
    S2 = torch.randn(5, H, dk, dk, generator=g) * 0.1
    _close(_both(lambda sb, a, b, c, d, e, f, st: sops.rwkv_time_mix(
        a, b, c, d, e, f, st, sb, H), [r, k, v, wr, w0, u], states=[S2]),
        atol=1e-4)

    P = 2 * H * dk + H * dv + 2 * H + 5
    pj = torch.randn(T, P, generator=g)
    offs = (3, 3 + H * dk, 3 + 2 * H * dk, 3 + 2 * H * dk + H * dv,
            3 + 2 * H * dk + H * dv + H)
    ib, fb = torch.randn(H, generator=g), torch.randn(H, generator=g) + 2
    Sm = torch.randn(5, H, dk, dv, generator=g) * 0.1
    n = torch.randn(5, H, dk, generator=g) * 0.1
    m = torch.rand(5, H, generator=g)
    _close(_both(lambda sb, p, a, b, s1, s2, s3: sops.mlstm_memory(
        p, offs, a, b, s1, s2, s3, sb, H, dv, dk ** -0.5, 8.0),
        [pj, ib, fb], states=[Sm, n, m]), atol=1e-4)


@pytest.mark.parametrize("H,G,dk,dv,ps", [(6, 3, 24, 40, 16), (3, 1, 10, 7, 8),
                                          (8, 2, 128, 128, 64),
                                          (4, 4, 64, 300, 16),
                                          (4, 2, 96, 96, 16),
                                          (2, 1, 200, 64, 64),
                                          (2, 2, 40, 256, 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention(H, G, dk, dv, ps, dtype):
    g = torch.Generator().manual_seed(3)
    spans = [(70, 0, 0), (1, 1, 130), (9, 2, 57)]
    pages_per = 140 // ps + 1
    P = 3 * pages_per + 2
    perm = torch.randperm(P, generator=g)[:3 * pages_per].view(3, pages_per)
    kc = torch.randn(P, G, ps, dk, generator=g).to(dtype)
    vc = torch.randn(P, G, ps, dv, generator=g).to(dtype)
    T = sum(s[0] for s in spans)
    proj = torch.randn(T, H * dk + G * (dk + dv) + 4, generator=g).to(dtype)
    pos, slots = [], []
    for i, (n, _s, p0) in enumerate(spans):
        for p in range(p0, p0 + n):
            pos.append(p)
            slots.append(int(perm[i, p // ps]) * ps + p % ps)
    r1, r2 = torch.rand(H, generator=g) * 2, torch.rand(H, generator=g) * 0.3
    outs = []
    for dev in ("cpu", DEV):
        sb, _ = _batch(spans, dev)
        sb.page_table = perm.to(torch.int32).to(dev)
        k_, v_ = kc.clone().to(dev), vc.clone().to(dev)
        pj = proj.to(dev)
        positions = torch.tensor(pos, dtype=torch.int32, device=dev)
        sm = torch.tensor(slots, dtype=torch.int64, device=dev)
        sops.kv_append_norm(k_, v_, pj, H * dk, H * dk + G * dk, sm, True, 1e-5)
        o = sops.biased_attention(pj, 0, H, k_, v_, positions, sb,
                                  r1.to(dev), r2.to(dev), 0.2, 0.7, 16)
        outs.append((o.float().cpu(), k_.float().cpu(), v_.float().cpu()))
    tol = 3e-5 if dtype == torch.float32 else 3e-2
    for a, b in zip(*outs):
        assert torch.allclose(a, b, atol=tol, rtol=1e-3), \
            float((a - b).abs().max())
    if dtype == torch.bfloat16 and sops.hip_seq().biased_attention_mfma_supported(dk, dv):
        # the matrix-core kernel on the same cache: the 70-row and 9-row
        # portions as tiles (64 + 6, 9), the single row on the row kernel
        # in between; against the row kernel it differs only by the bf16
        # rounding of the softmax weights
        order = [1, 0, 2]                      # decoded row first
        spans2 = [spans[i] for i in order]
        sb, _ = _batch(spans2, DEV)
        sb.page_table = perm[order].to(torch.int32).to(DEV)
        rows = torch.cat([torch.arange(70, 71), torch.arange(0, 70),
                          torch.arange(71, 80)])
        sb.num_decode = 1
        sb.tiles = (torch.tensor([1, 65, 71], dtype=torch.int32, device=DEV),
                    torch.tensor([64, 6, 9], dtype=torch.int32, device=DEV))
        o2 = sops.biased_attention(
            proj[rows].to(DEV), 0, H, k_, v_,
            torch.tensor(pos, dtype=torch.int32)[rows].to(DEV), sb,
            r1.to(DEV), r2.to(DEV), 0.2, 0.7, 16).float().cpu()
        ref = outs[1][0][rows]
        assert torch.allclose(o2, ref, atol=2e-2, rtol=2e-2), \
            float((o2 - ref).abs().max())
