"""Each HIP kernel alone against its plain reference, at other sizes than the engine's tiny
models use, in 32-bit and in bfloat16, with inputs made so that a fault shows (a far key that
must win, a window's edge, scattered page ids)."""
import math
import os

import numpy as np
import pytest
import torch

import plain_gemma3 as P

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DEV = "cuda:0"


def _g(name):
    path = os.path.join(GOLDEN, name + ".bin")
    if not os.path.isfile(path):
        pytest.skip("reference golden vectors not mounted")
    return torch.from_numpy(np.fromfile(path, dtype="<f4").copy())


def _i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def _tol(dtype):
    return dict(atol=2e-6, rtol=2e-6) if dtype == torch.float32 else dict(atol=1e-2, rtol=1e-2)


@pytest.fixture(scope="module")
def K():
    from agave_amd.ops import kernels
    return kernels


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_scale(K, dtype):
    table = (torch.randn(300, 72) * 0.05).to(dtype)
    toks = [0, 299, 17, 17, 123]
    out = torch.empty(5, 72, dtype=torch.float32, device=DEV)
    K.embed_scale(_i32(toks), table.to(DEV), math.sqrt(72.0), out)
    ref = P.embed(toks, table.double(), 72)
    assert torch.allclose(out.cpu().double(), ref, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("e", [100, 2560, 3136])
def test_residual_norm(K, dtype, e):
    n = 7
    h = torch.randn(n, e) * 3
    br = (torch.randn(n, e) * 0.3).to(dtype)
    gp, gq = torch.randn(e) * 0.1 + 1, torch.randn(e) * 0.1 + 1
    hd = h.clone().to(DEV)
    out = torch.empty(n, e, dtype=dtype, device=DEV)
    K.residual_norm(hd, br.to(DEV), gp.to(DEV), 1e-5, out, gq.to(DEV), 3e-6)
    h_ref = h.double() + P.rms_norm(br.double(), gp.double(), 1e-5, add_one=False)
    o_ref = P.rms_norm(h_ref, gq.double(), 3e-6, add_one=False)
    assert torch.allclose(hd.cpu().double(), h_ref, atol=3e-6, rtol=1e-6)      # the sum is 32-bit in both types
    assert torch.allclose(out.cpu().double(), o_ref, **_tol(dtype))
    # norm only, on gathered rows; and a plain add without a norm on the branch
    rows = _i32([5, 0, 5])
    out2 = torch.empty(3, e, dtype=dtype, device=DEV)
    K.residual_norm(hd, None, None, 0.0, out2, gq.to(DEV), 3e-6, rows)
    assert torch.allclose(out2.cpu().double(), o_ref[[5, 0, 5]], **_tol(dtype))
    h3 = h.clone().to(DEV)
    K.residual_norm(h3, br.to(DEV), None, 0.0, None, None, 0.0)
    assert torch.allclose(h3.cpu().double(), h.double() + br.double(), atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("e", [100, 2560, 20000])
def test_residual_norm_reads_the_stream_elsewhere(K, dtype, e):
    """``src``: the residual rows are read from another tensor and written to h, with a branch, with
    slices, with a norm only and with nothing else to do (both kernels: 20,000 columns are too many
    for the one that holds a row in registers)."""
    n = 4
    src = torch.randn(n, e) * 3
    br = (torch.randn(n, e) * 0.3).to(dtype)
    parts = torch.randn(3, n, e) * 0.3
    gp, gq = torch.randn(e) * 0.1 + 1, torch.randn(e) * 0.1 + 1
    for branch, b_sum in ((br, br.double()), (parts, parts.double().sum(0)), (None, None)):
        h = torch.full((n, e), 9.0, device=DEV)
        s_dev = src.clone().to(DEV)
        out = torch.empty(n, e, dtype=dtype, device=DEV)
        K.residual_norm(h, branch.to(DEV) if branch is not None else None, gp.to(DEV) if branch is not None else None, 1e-5,
                        out, gq.to(DEV), 3e-6, src=s_dev)
        h_ref = src.double() + (P.rms_norm(b_sum, gp.double(), 1e-5, add_one=False) if b_sum is not None else 0.0)
        assert torch.allclose(h.cpu().double(), h_ref, atol=3e-6, rtol=1e-6)
        assert torch.allclose(out.cpu().double(), P.rms_norm(h_ref, gq.double(), 3e-6, add_one=False), **_tol(dtype))
        assert torch.equal(s_dev.cpu(), src)
    h = torch.full((n, e), 9.0, device=DEV)
    K.residual_norm(h, br.to(DEV), None, 0.0, None, None, 0.0, src=src.to(DEV))         # a plain add
    assert torch.allclose(h.cpu().double(), src.double() + br.double(), atol=1e-6)
    K.residual_norm(h, None, None, 0.0, None, None, 0.0, src=src.to(DEV))               # nothing but the move
    assert torch.equal(h.cpu(), src)
    with pytest.raises(ValueError):
        K.residual_norm(h, None, None, 0.0, None, None, 0.0, src=h)
    with pytest.raises(ValueError):
        K.residual_norm(h, None, None, 0.0, torch.empty(1, e, dtype=dtype, device=DEV), gq.to(DEV), 1e-6, _i32([1]), src=src.to(DEV))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("e", [72, 2560, 5000])
def test_residual_norm_takes_a_branch_in_slices(K, dtype, e):
    """A float32 [slices, rows, hidden] branch stands for the sum of its slices: the same residual
    stream and output as with the sum given as one 32-bit branch (both row-in-registers and plain kernel)."""
    n, slices = 5, 3
    h = torch.randn(n, e) * 3
    parts = torch.randn(slices, n, e) * 0.3
    gp, gq = torch.randn(e) * 0.1 + 1, torch.randn(e) * 0.1 + 1
    hd = h.clone().to(DEV)
    out = torch.empty(n, e, dtype=dtype, device=DEV)
    K.residual_norm(hd, parts.to(DEV), gp.to(DEV), 1e-5, out, gq.to(DEV), 3e-6)
    h_ref = h.double() + P.rms_norm(parts.double().sum(0), gp.double(), 1e-5, add_one=False)
    o_ref = P.rms_norm(h_ref, gq.double(), 3e-6, add_one=False)
    assert torch.allclose(hd.cpu().double(), h_ref, atol=3e-6, rtol=1e-6)
    assert torch.allclose(out.cpu().double(), o_ref, **_tol(dtype))
    h3 = h.clone().to(DEV)
    K.residual_norm(h3, parts.to(DEV), None, 0.0, None, None, 0.0)           # a plain add of the slices
    assert torch.allclose(h3.cpu().double(), h.double() + parts.double().sum(0), atol=2e-6)
    with pytest.raises(ValueError):
        K.residual_norm(h3, parts[:, :4].to(DEV), None, 0.0, None, None, 0.0)


@pytest.mark.parametrize("n", [128, 1152, 2560, 3136])
def test_residual_norm_golden(K, n):
    # research/kernels/generate_golden.py:98-110 (eps 1e-5, plain weight)
    x, w, want = _g(f"rms_norm_n{n}_x"), _g(f"rms_norm_n{n}_w"), _g(f"rms_norm_n{n}_out")
    h = x.view(1, n).clone().to(DEV)
    out = torch.empty(1, n, dtype=torch.float32, device=DEV)
    K.residual_norm(h, None, None, 0.0, out, w.to(DEV), 1e-5)
    assert torch.allclose(out.cpu().view(-1), want, atol=2e-5, rtol=1e-5)


def _pages(n_pages, nkv, hd, dtype):
    k = torch.zeros(n_pages, nkv, 64, hd, dtype=dtype, device=DEV)
    v = torch.zeros(n_pages, nkv, hd, 64, dtype=dtype, device=DEV)
    return k, v


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_qk_norm_rope_kv(K, dtype):
    nh, nkv, hd, rot = 3, 1, 40, 24           # head size no multiple of 16, partial rotation
    seqs = [(0, 5, 3), (1, 130, 4)]           # (sequence, first position, tokens)
    tok_seq = [b for b, _, n in seqs for _ in range(n)]
    tok_pos = [p + i for _, p, n in seqs for i in range(n)]
    n = len(tok_pos)
    q = (torch.randn(n, nh * hd)).to(dtype)
    k = (torch.randn(n, nkv * hd)).to(dtype)
    v = (torch.randn(n, nkv * hd)).to(dtype)
    qg, kg = torch.randn(hd) * 0.1 + 1, torch.randn(hd) * 0.1 + 1
    inv = torch.from_numpy(np.exp(-np.log(5e3) * 2.0 * np.arange(rot // 2) / rot).astype(np.float32))
    kp, vp = _pages(6, nkv, hd, dtype)
    table = _i32([[4, -1, -1], [-1, 5, 2]])   # sequence 1: base 1, so page index 2 is column 1 -> page 5
    base = _i32([0, 1])
    q_out = torch.empty(n, nh * hd, dtype=dtype, device=DEV)
    K.qk_norm_rope_kv(q.to(DEV), k.to(DEV), v.to(DEV), q_out, qg.to(DEV), kg.to(DEV), 1e-6, 2e-6, inv.to(DEV), 0.25,
                      _i32(tok_seq), _i32(tok_pos), kp, vp, table, base, nh, nkv, hd)
    pos = torch.tensor(tok_pos, dtype=torch.float64)
    ang = P.rope_angles(pos, rot, 5e3, 4.0)
    q_ref = P.apply_rope(P.rms_norm(q.double().view(n, nh, hd), qg.double(), 1e-6, add_one=False), ang)
    k_ref = P.apply_rope(P.rms_norm(k.double().view(n, nkv, hd), kg.double(), 2e-6, add_one=False), ang)
    tol = dict(atol=3e-6, rtol=3e-6) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)
    assert torch.allclose(q_out.cpu().double().view(n, nh, hd), q_ref, **tol)
    page_of = {0: {0: 4}, 1: {2: 5}}
    for t, (b, p) in enumerate(zip(tok_seq, tok_pos)):
        pg, row = page_of[b][p // 64], p % 64
        assert torch.allclose(kp[pg, :, row, :].cpu().double(), k_ref[t], **tol)
        assert torch.equal(vp[pg, :, :, row].cpu().view(-1), v[t])            # v is stored as it is
    # rows that no token wrote stay zero
    written = {(page_of[b][p // 64], p % 64) for b, p in zip(tok_seq, tok_pos)}
    mask = torch.ones(6, 64, dtype=torch.bool)
    for pg, row in written:
        mask[pg, row] = False
    assert float(kp.cpu().float().abs().sum(dim=(1, 3))[mask].sum()) == 0.0


@pytest.mark.parametrize("pos", [0, 1, 10, 100, 1000])
def test_rope_golden(K, pos):
    # research/kernels/generate_golden.py:140-155: nh 4, hd 256, theta 1e4, no norm
    q, want = _g(f"rope_nh4_hd256_pos{pos}_q_in"), _g(f"rope_nh4_hd256_pos{pos}_q_out")
    inv = torch.from_numpy(np.exp(-np.log(1e4) * 2.0 * np.arange(128) / 256).astype(np.float32))
    q_out = torch.empty(1, 1024, dtype=torch.float32, device=DEV)
    K.qk_norm_rope_kv(q.view(1, -1).to(DEV), None, None, q_out, None, None, 0.0, 0.0, inv.to(DEV), 1.0,
                      _i32([0]), _i32([pos]), None, None, None, None, 4, 0, 256)
    assert torch.allclose(q_out.cpu().view(-1), want, atol=3e-4 if pos >= 100 else 2e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_geglu(K, dtype):
    n, ff = 5, 333
    gu = (torch.randn(n, 2 * ff) * 2).to(dtype).to(DEV)
    out = torch.empty(n, ff, dtype=dtype, device=DEV)
    K.geglu(gu[:, :ff], gu[:, ff:], out)
    ref = P.gelu_tanh(gu[:, :ff].cpu().double()) * gu[:, ff:].cpu().double()
    assert torch.allclose(out.cpu().double(), ref, **_tol(dtype))
    big = torch.tensor([[-100.0, 100.0, 1.0, 1.0]], device=DEV)
    o = torch.empty(1, 2, device=DEV)
    K.geglu(big[:, :2], big[:, 2:], o)
    assert torch.isfinite(o).all() and float(o[0, 1]) == 100.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("activation", ["gelu_tanh", "silu", "gelu", "relu"])
def test_gated_act_takes_the_activation_as_a_parameter(K, dtype, activation):
    """out = act(gate) * up for every activation the kernel knows, against the library's functions
    in 64-bit; large arguments of either sign stay finite."""
    n, ff = 7, 301
    gu = (torch.randn(n, 2 * ff, generator=torch.Generator().manual_seed(5)) * 3).to(dtype)
    gu[0, :4] = torch.tensor([-90.0, 90.0, -30.0, 30.0]).to(dtype)
    out = torch.full((n, ff), float("nan"), dtype=dtype, device=DEV)
    K.gated_act(gu[:, :ff].to(DEV), gu[:, ff:].to(DEV), out, activation)
    g, u = gu[:, :ff].double(), gu[:, ff:].double()
    act = {"gelu_tanh": P.gelu_tanh, "silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu,
           "relu": torch.relu}[activation]
    assert torch.isfinite(out.float()).all()
    assert torch.allclose(out.cpu().double(), act(g) * u, **_tol(dtype))
    with pytest.raises(ValueError, match="unknown activation"):
        K.gated_act(gu[:, :ff].to(DEV), gu[:, ff:].to(DEV), out, "swish_of_tomorrow")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_add_bias_to_rows_of_a_wider_matrix(K, dtype):
    """y[r] += bias, summed in 32-bit and rounded once; the columns beside the rows' stretch stay."""
    n, cols = 9, 203
    g = torch.Generator().manual_seed(6)
    wide = torch.randn(n, cols + 13, generator=g).to(dtype).to(DEV)
    before = wide.clone()
    bias = torch.randn(cols, generator=g).to(DEV)
    K.add_bias(wide[:, 5:5 + cols], bias)
    want = (before[:, 5:5 + cols].float() + bias).to(dtype)
    assert torch.equal(wide[:, 5:5 + cols], want)
    assert torch.equal(wide[:, :5], before[:, :5]) and torch.equal(wide[:, 5 + cols:], before[:, 5 + cols:])
    with pytest.raises(TypeError):
        K.add_bias(wide[:, 5:5 + cols], bias[:-1])


@pytest.mark.parametrize("scale,cap", [(1.0, 30.0), (2.5, 4.0), (0.125, 0.0)])
def test_scale_and_soft_cap_of_logits(K, scale, cap):
    """x <- cap tanh(scale x / cap), or scale x without a cap; huge logits end at the cap, not at NaN."""
    x = torch.randn(5, 1001, generator=torch.Generator().manual_seed(7)) * 6
    x[0, :3] = torch.tensor([1e6, -1e6, 0.0])
    y = x.to(DEV)
    K.scale_cap(y, scale, cap)
    want = x.double() * scale
    if cap > 0:
        want = cap * torch.tanh(want / cap)
    assert torch.isfinite(y).all()
    assert torch.allclose(y.cpu().double(), want, atol=2e-6 * max(cap, 1.0), rtol=2e-6)
    with pytest.raises(ValueError):
        K.scale_cap(y, 1.0, -1.0)


@pytest.mark.parametrize("n", [128, 1152, 6912])
def test_gelu_golden(K, n):
    x, want = _g(f"gelu_n{n}_x"), _g(f"gelu_n{n}_out")
    out = torch.empty(1, n, device=DEV)
    K.geglu(x.view(1, n).to(DEV), torch.ones(1, n, device=DEV), out)
    assert torch.allclose(out.cpu().view(-1), want, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("ta,tw,tc", [(torch.float32,) * 3, (torch.bfloat16,) * 3,
                                      (torch.bfloat16, torch.bfloat16, torch.float32),
                                      (torch.bfloat16, torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("m,n,k", [(1, 53, 29), (37, 130, 75), (65, 64, 16)])
def test_gemm_plain(K, ta, tw, tc, m, n, k):
    a, w = torch.randn(m, k).to(ta), torch.randn(n, k).to(tw)
    c = torch.empty(m, n, dtype=tc, device=DEV)
    K.gemm_plain(a.to(DEV), w.to(DEV), c)
    ref = a.double() @ w.double().T
    tol = dict(atol=1e-5, rtol=1e-5) if tc == torch.float32 else dict(atol=5e-2, rtol=1e-2)
    assert torch.allclose(c.cpu().double(), ref, **tol)
    # a strided input (a slice of a wider matrix)
    wide = torch.randn(m, k + 11).to(ta).to(DEV)
    K.gemm_plain(wide[:, 5:5 + k], w.to(DEV), c)
    assert torch.allclose(c.cpu().double(), wide[:, 5:5 + k].cpu().double() @ w.double().T, **tol)


def _attn_case(K, dtype, nh, nkv, hd, lens, window, scale, seed=0, boost=None):
    """Sequences of the given lengths in scattered pages; every position is a query."""
    g = torch.Generator().manual_seed(seed)
    n_pages = sum((L + 63) // 64 for L in lens) + 3
    kp, vp = _pages(n_pages, nkv, hd, dtype)
    perm = torch.randperm(n_pages, generator=g).tolist()
    width = max((L + 63) // 64 for L in lens)
    table = torch.full((len(lens), width), -1, dtype=torch.int32)
    ks, vs, qs, tok_seq, tok_pos = [], [], [], [], []
    for b, L in enumerate(lens):
        k = torch.randn(L, nkv, hd, generator=g).to(dtype)
        v = torch.randn(L, nkv, hd, generator=g).to(dtype)
        q = torch.randn(L, nh, hd, generator=g).to(dtype)
        if boost is not None:                  # one far key must win for the last query:
            k = k - k.mean(dim=-1, keepdim=True)   # every other key is orthogonal to that query (score 0),
            k[boost] = 1.0                         # the far key scores 20
            q[L - 1] = 20.0 / (hd * scale)
        for i in range((L + 63) // 64):
            pg = perm.pop()
            table[b, i] = pg
            rows = slice(i * 64, min(L, i * 64 + 64))
            kp[pg, :, :rows.stop - rows.start, :] = k[rows].transpose(0, 1).to(DEV)
            vp[pg, :, :, :rows.stop - rows.start] = v[rows].permute(1, 2, 0).to(DEV)
        ks.append(k); vs.append(v); qs.append(q)
        tok_seq += [b] * L
        tok_pos += list(range(L))
    q_all = torch.cat(qs).reshape(-1, nh * hd).to(DEV)
    out = torch.empty_like(q_all)
    K.attn_plain(q_all, out, kp, vp, table.to(DEV), _i32([0] * len(lens)), _i32(tok_seq), _i32(tok_pos),
                 nh, nkv, hd, scale, window)
    refs = [P.attention_core(q.double(), k.double(), v.double(), scale, window) for q, k, v in zip(qs, ks, vs)]
    return out.cpu().double().view(-1, nh, hd), torch.cat(refs), vs


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 40, None), (6, 1, 16, 70), (5, 5, 72, 300), (2, 1, 256, 64)])
def test_attn_plain(K, dtype, nh, nkv, hd, window):
    got, ref, _ = _attn_case(K, dtype, nh, nkv, hd, [1, 77, 300, 64], window, 0.21)
    # 32-bit: a score is a sum of hd products of N(0,1) values, so its rounding error, and with it
    # the relative error of exp(score), grows with hd
    tol = dict(atol=2e-6 + 1e-7 * hd, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    assert torch.allclose(got, ref, **tol)


def test_attn_plain_far_key_wins(K):
    # among 700 keys, key 3 is made to dominate the last query's softmax: the output must be its value
    got, ref, vs = _attn_case(K, torch.float32, 2, 1, 32, [700], None, 0.5, seed=1, boost=3)
    assert torch.allclose(got[-1], ref[-1], atol=1e-5)
    assert torch.allclose(got[-1, 0], vs[0][3, 0].double(), atol=1e-2)
    # with a window that ends before it, the same key must not be seen
    got_w, ref_w, _ = _attn_case(K, torch.float32, 2, 1, 32, [700], 696, 0.5, seed=1, boost=3)
    assert torch.allclose(got_w[-1], ref_w[-1], atol=1e-5)
    assert not torch.allclose(got_w[-1, 0], vs[0][3, 0].double(), atol=1e-1)
    got_e, ref_e, _ = _attn_case(K, torch.float32, 2, 1, 32, [700], 697, 0.5, seed=1, boost=3)   # edge: just inside
    assert torch.allclose(got_e[-1, 0], vs[0][3, 0].double(), atol=1e-2)


@pytest.mark.parametrize("tag,nh,nkv,hd,sl,suffix", [
    ("sdpa_nh4_nkv1_hd256_sl256", 4, 1, 256, 256, "_naive"), ("sdpa_nh4_nkv1_hd256_sl64", 4, 1, 256, 64, "_online"),
    ("sdpa_nh20_nkv5_hd128_sl32", 20, 5, 128, 32, ""), ("sdpa_nh4_nkv1_hd256_sl1", 4, 1, 256, 1, "_naive")])
def test_attn_plain_golden(K, tag, nh, nkv, hd, sl, suffix):
    # research/kernels/generate_golden.py:56-95; the reference's criterion is max error < 1e-3
    # (tests/sdpa_harness.zig:124-136); 32-bit sums give far less
    q, keys, values = _g(tag + "_q"), _g(tag + "_keys").view(sl, nkv, hd), _g(tag + "_values").view(sl, nkv, hd)
    n_pages = (sl + 63) // 64
    kp, vp = _pages(n_pages, nkv, hd, torch.float32)
    for i in range(n_pages):
        rows = slice(i * 64, min(sl, i * 64 + 64))
        kp[i, :, :rows.stop - rows.start] = keys[rows].transpose(0, 1).to(DEV)
        vp[i, :, :, :rows.stop - rows.start] = values[rows].permute(1, 2, 0).to(DEV)
    out = torch.empty(1, nh * hd, device=DEV)
    K.attn_plain(q.view(1, -1).to(DEV), out, kp, vp, _i32([list(range(n_pages))]), _i32([0]), _i32([0]), _i32([sl - 1]),
                 nh, nkv, hd, 1.0 / math.sqrt(hd), None)
    assert torch.allclose(out.cpu().view(-1), _g(tag + "_out" + suffix), atol=2e-5)


# ---------------------------------------------------------------- sampling
@pytest.fixture(scope="module")
def S():
    from agave_amd.ops import sampling
    return sampling


def _sample(S, logits, params):
    lg = logits.to(DEV).float().contiguous()
    work = torch.empty_like(lg)
    out = torch.empty(lg.shape[0], dtype=torch.int32, device=DEV)
    S.sample(lg, work, torch.tensor(params, dtype=torch.float32, device=DEV), out)
    got = out.cpu().tolist()
    # with scratch, rows of a large vocabulary are shared among workgroups; what it held before must not matter
    class Row:
        def __init__(self, p):
            self.temperature, self.top_k, self.top_p = p[0], int(p[1]), p[2]
    for kinds in (S.KIND_ALL, S.kinds_of([Row(p) for p in params], lg.shape[1])):
        scratch = torch.randint(-2 ** 31, 2 ** 31 - 1, (S.scratch_words() * lg.shape[0],), dtype=torch.int32,
                                device=DEV).view(torch.float32)
        out.fill_(-1)
        S.sample(lg, work, torch.tensor(params, dtype=torch.float32, device=DEV), out, scratch, kinds=kinds)
        assert out.cpu().tolist() == got
    return got


def test_argmax_first_of_ties(S):
    lg = torch.full((3, 5000), -1.0)
    lg[0, [4000, 77, 3000]] = 2.0
    lg[1, :] = float("-inf")
    lg[2, 4999] = 0.5
    assert _sample(S, lg, [[0, 0, 1, 0.9]] * 3) == [77, 0, 4999]


@pytest.mark.parametrize("temperature,top_k,top_p", [(1.0, 0, 1.0), (0.7, 0, 1.0), (1.3, 5, 1.0), (1.0, 0, 0.6),
                                                      (0.9, 50, 0.8), (1.0, 2000, 0.95), (2.0, 1, 1.0)])
@pytest.mark.parametrize("vocab", [3001, 40013, 262208])
def test_sample_matches_plain_rule(S, temperature, top_k, top_p, vocab):
    """For every token the plain rule can draw, a u in the middle of its interval of the running
    sum must give exactly that token."""
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(vocab, generator=g) * 2.5
    w = P.sample_distribution(logits, temperature, top_k, top_p)
    cdf = torch.cumsum(w, 0) / w.sum()
    support = torch.nonzero(w > 0).view(-1).tolist()
    if top_k:
        assert len(support) <= min(top_k, 1024)
    picks = support if len(support) <= 64 else [support[i] for i in range(0, len(support), len(support) // 64)]
    us, want = [], []
    for i in picks:
        lo = float(cdf[i - 1]) if i > 0 else 0.0
        hi = float(cdf[i])
        if hi - lo < 1e-5:
            continue
        us.append((lo + hi) / 2)
        want.append(i)
    got = _sample(S, logits.view(1, -1).repeat(len(us), 1), [[temperature, top_k, top_p, u] for u in us])
    assert got == want
    assert all(P.sample_token(logits, temperature, top_k, top_p, u) == i for u, i in zip(us, want))


def test_sample_rows_are_independent_and_mixed(S):
    g = torch.Generator().manual_seed(6)
    lg = torch.randn(4, 70001, generator=g)
    params = [[0.0, 0, 1.0, 0.3], [0.8, 0, 1.0, 0.3], [0.8, 3, 1.0, 0.99], [1.0, 0, 0.5, 0.0]]
    together = _sample(S, lg, params)
    alone = [_sample(S, lg[i:i + 1], [params[i]])[0] for i in range(4)]
    assert together == alone
    assert together[0] == int(lg[0].argmax())
    assert together[2] in torch.topk(lg[2], 3).indices.tolist()
    assert together == [P.sample_token(lg[i], *params[i]) for i in range(4)]


@pytest.mark.parametrize("vocab", [3001, 4096, 40013])
@pytest.mark.parametrize("temperature,top_k,top_p", [(0.8, 0, 0.01), (1.7, 5000, 0.01), (1.0, 1000, 1.0),
                                                      (0.8, 0, 0.9), (1.3, 1024, 0.7), (1.0, 900, 0.5)])
def test_sample_with_more_equal_logits_than_the_filter_collects(S, vocab, temperature, top_k, top_p):
    """Some hundred logits above a plateau of far more than a thousand equal ones: the 1024 largest
    end inside the plateau, all of which stays or goes together, and the draw has to range over
    entries that the filter could not collect.  top_p = 0.01 keeps the maximum alone: its weight,
    which is exactly 1, has to equal the threshold wherever it is computed again."""
    g = torch.Generator().manual_seed(vocab + top_k)
    logits = torch.randn(vocab, generator=g) * 2.0
    plateau = float(torch.sort(logits, descending=True).values[700])
    logits[::3] = plateau                                  # vocab / 3 equal entries below about 470 others
    w = P.sample_distribution(logits, temperature, top_k, top_p)
    cdf = torch.cumsum(w, 0) / w.sum()
    support = torch.nonzero(w > 0).view(-1).tolist()
    picks = support if len(support) <= 48 else [support[i] for i in range(0, len(support), len(support) // 48)]
    picks = sorted(set(picks + support[-2:]))
    us, want = [], []
    for i in picks:
        lo = float(cdf[i - 1]) if i > 0 else 0.0
        hi = float(cdf[i])
        if hi - lo < 1e-5:
            continue
        us.append((lo + hi) / 2)
        want.append(i)
    assert us
    got = _sample(S, logits.view(1, -1).repeat(len(us), 1), [[temperature, top_k, top_p, u] for u in us])
    assert got == want


def test_sample_random_parameters_ties_and_masked_halves(S):
    """A sweep of random rows and parameters, some rows with a seventh of their entries equal and
    some with their upper half at -inf, six rows a batch with mixed kinds; every draw must be the
    plain rule's (a u within 1e-4 of an interval's edge may go to the neighbour)."""
    rng = np.random.default_rng(0)
    checked = 0
    for trial in range(48):
        vocab = int(rng.choice([4096, 5003, 40013]))
        g = torch.Generator().manual_seed(trial)
        lg = torch.randn(6, vocab, generator=g) * float(rng.choice([0.5, 2.0, 6.0]))
        if trial % 3 == 0:
            lg[:, ::7] = lg[:, 3:4]
        if trial % 4 == 0:
            lg[:, vocab // 2:] = float("-inf")
        params = [[float(rng.choice([0.0, 0.3, 0.8, 1.0, 1.7])), int(rng.choice([0, 0, 1, 5, 40, 1000, 1024, 5000])),
                   float(rng.choice([1.0, 1.0, 0.95, 0.7, 0.3, 0.01])), float(rng.random())] for _ in range(6)]
        got = _sample(S, lg, params)
        for b, (t, k, p, u) in enumerate(params):
            want = P.sample_token(lg[b], t, k, p, u)
            if got[b] != want:
                w = P.sample_distribution(lg[b], t, k, p)
                assert t > 0 and float(w[got[b]]) > 0, (trial, b, params[b], got[b], want)
                cdf = torch.cumsum(w, 0) / w.sum()
                edges = [float(cdf[got[b]])] + ([float(cdf[got[b] - 1])] if got[b] else [])
                assert min(abs(e - u) for e in edges) < 1e-4, (trial, b, params[b], got[b], want)
            checked += 1
    assert checked == 48 * 6


def test_sample_frequencies_follow_softmax(S):
    lg = torch.tensor([[0.0, 1.0, 2.0, -1.0, 0.5]])
    n = 4000
    us = (torch.arange(n) + 0.5) / n                    # a stratified sweep of u
    got = _sample(S, lg.repeat(n, 1), [[0.7, 0, 1.0, float(u)] for u in us])
    freq = torch.bincount(torch.tensor(got), minlength=5).double() / n
    assert torch.allclose(freq, torch.softmax(lg[0].double() / 0.7, 0), atol=2.0 / n)


def test_repeat_penalty(S):
    lg = torch.tensor([[2.0, -2.0, 1.0, 3.0], [2.0, -2.0, 1.0, 3.0], [1.0, 1.0, 1.0, 1.0]], device=DEV)
    ids = _i32([0, 1, 0, 9, 3])
    cu = _i32([0, 4, 5, 5])
    S.repeat_penalty(lg, ids, cu, torch.tensor([2.0, 3.0, 1.5], device=DEV))
    want = torch.stack([P.apply_repeat_penalty(torch.tensor([2.0, -2.0, 1.0, 3.0]), [0, 1, 0, 9], 2.0),
                        P.apply_repeat_penalty(torch.tensor([2.0, -2.0, 1.0, 3.0]), [3], 3.0),
                        torch.ones(4)])
    assert torch.allclose(lg.cpu(), want, atol=1e-6)


def test_cpu_tensors_are_refused(K):
    with pytest.raises(RuntimeError, match="GPU"):
        K.gemm_plain(torch.zeros(2, 2), torch.zeros(2, 2), torch.zeros(2, 2))


# ---------------------------------------------------------------- matrix-core products
@pytest.mark.parametrize("b,v", [(1, 7), (5, 1000), (8, 262208), (3, 4099)])
def test_token_logprob(S, b, v):
    """log softmax at one entry of each row, rows with -inf entries and a row strides apart among them."""
    g = torch.Generator().manual_seed(b + v)
    wide = (torch.randn(b, v + 5, generator=g) * 4).to(DEV)
    logits = wide[:, :v]
    logits[0, : v // 2] = float("-inf")
    toks = torch.randint(v // 2, v, (b,), generator=g).to(torch.int32).to(DEV)
    out = torch.full((b,), float("nan"), device=DEV)
    S.token_logprob(logits, toks, out)
    ref = torch.log_softmax(logits.double(), -1)[torch.arange(b), toks.long()]
    assert torch.allclose(out.double(), ref, atol=2e-5, rtol=0)
    if v > 2:                                               # an entry that is -inf has probability 0
        S.token_logprob(logits, torch.zeros(b, dtype=torch.int32, device=DEV), out)
        assert float(out[0]) == float("-inf")


@pytest.fixture(scope="module")
def G():
    from agave_amd.ops import gemm_mfma
    return gemm_mfma


@pytest.mark.parametrize("m", [1, 3, 16, 17, 40, 64])
@pytest.mark.parametrize("n,k", [(53, 72), (256, 2560), (1000, 96), (4100, 136), (160, 10240)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_gemm_skinny(G, m, n, k, out_dtype):
    g = torch.Generator().manual_seed(m * 1000 + n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
    packed = G.pack_weight(w.to(DEV))
    out = torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)
    G.skinny(x.to(DEV), packed, out, n)
    ref = x.double() @ w.double().T
    scale = float(ref.abs().max())
    tol = 2e-5 * scale * math.sqrt(k / 64) if out_dtype == torch.float32 else 6e-3 * scale
    assert float((out.cpu().double() - ref).abs().max()) <= tol


@pytest.mark.parametrize("m,ff,k", [(1, 192, 64), (8, 1000, 96), (33, 10240, 256), (64, 20, 40)])
def test_gemm_skinny_geglu(G, m, ff, k):
    g = torch.Generator().manual_seed(ff + m)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(2 * ff, k, generator=g) * 0.2).bfloat16()
    packed = G.pack_weight(w.to(DEV), interleave_ff=ff)
    out = torch.full((m, ff), float("nan"), dtype=torch.bfloat16, device=DEV)
    G.skinny(x.to(DEV), packed, out, ff, epilogue=1)
    gu = x.double() @ w.double().T
    ref = P.gelu_tanh(gu[:, :ff]) * gu[:, ff:]
    assert float((out.cpu().double() - ref).abs().max()) <= 8e-3 * float(ref.abs().max())


@pytest.mark.parametrize("m,n,k,slices", [(8, 160, 10240, 3), (1, 53, 4104, 2), (16, 256, 2560, 5), (40, 100, 1096, 2)])
def test_gemm_skinny_in_slices(G, m, n, k, slices):
    """The product shared out along its columns: the 32-bit slices add up to it; runs of columns of
    unequal length, and a last one that ends inside a tile."""
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
    packed = G.pack_weight(w.to(DEV))
    out = torch.full((slices, m, n), float("nan"), device=DEV)
    G.skinny_slices(x.to(DEV), packed, out, n)
    ref = x.double() @ w.double().T
    assert float((out.cpu().double().sum(0) - ref).abs().max()) <= 2e-5 * float(ref.abs().max()) * math.sqrt(k / 64)
    assert float(out[0].abs().max()) > 0 and float(out[-1].abs().max()) > 0
    with pytest.raises(ValueError):
        G.skinny_slices(x.to(DEV), packed, out.bfloat16(), n)
    assert G.slices_for(8, 2560, 10240) > 1 and G.slices_for(8, 10240, 2560) == 1 and G.slices_for(65, 2560, 10240) == 1


@pytest.mark.parametrize("m,n,k,epi", [(1, 4096, 2560, 0), (1, 10240, 2560, 1), (1, 1000, 5376, 1), (1, 53, 200, 0),
                                       (1, 40, 72, 1), (1, 130, 3080, 0), (1, 96, 6144, 0), (1, 8192, 3840, 0),
                                       (1, 21504, 5376, 1), (1, 4100, 4104, 0), (1, 40000, 64, 0), (1, 36, 72, 1),
                                       (1, 21, 40, 0)])
@pytest.mark.parametrize("branch", ["none", "bf16", "f32", "slices", "slices_unnormed", "slices11", "slices2"])
def test_product_of_one_token_that_makes_its_own_normalised_row(G, m, n, k, epi, branch):
    """out = rmsnorm(h + post(branch)) W^T (or its GeGLU) for one row, h + post(branch) going
    to other memory: against the same written out in 64-bit, with the normalised rows rounded to
    bfloat16 as the kernel rounds them.  The gains differ per column and the branch is large against
    h, so that a gain or a norm left out, or applied in the wrong place, shows; memory beside the
    outputs must stay as it was."""
    assert G.normed_ok(m, n, k, epi)
    g = torch.Generator().manual_seed(m * 7 + n + k + len(branch))
    h = torch.randn(m, k, generator=g) * 2
    pre_gain, post_gain = torch.rand(k, generator=g) + 0.5, torch.rand(k, generator=g) * 2 + 0.5
    pre_eps, post_eps = 1e-3, 0.5
    rows = 2 * n if epi else n
    w = (torch.randn(rows, k, generator=g) * 0.1).bfloat16()
    packed = G.pack_weight(w.to(DEV), interleave_ff=n if epi else 0)
    b = b_sum = None
    if branch == "bf16":
        b = (torch.randn(m, k, generator=g) * 5).bfloat16()
        b_sum = b.double()
    elif branch == "f32":
        b = torch.randn(m, k, generator=g) * 5
        b_sum = b.double()
    elif branch.startswith("slices"):
        # (two slices are asked for ahead of the weights, or eight when there are more than two; others follow)
        b = torch.randn({"slices11": 11, "slices2": 2}.get(branch, 5), m, k, generator=g) * 3
        b_sum = b.double().sum(0)
    with_post = branch not in ("none", "slices_unnormed")
    hd = h.double()
    if b_sum is not None:
        if with_post:
            hd = hd + b_sum / torch.sqrt((b_sum * b_sum).mean(-1, keepdim=True) + post_eps) * post_gain.double()
        else:
            hd = hd + b_sum
    x = (hd / torch.sqrt((hd * hd).mean(-1, keepdim=True) + pre_eps) * pre_gain.double()).bfloat16().double()
    y = x @ w.double().T
    ref = P.gelu_tanh(y[:, :n]) * y[:, n:] if epi else y

    h_dev = h.to(DEV)
    h_out = torch.full((m + 1, k), 7.0, device=DEV)
    out = torch.full((m + 1, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    G.row_normed(h_dev, h_out[:m] if b is not None else None, b.to(DEV) if b is not None else None,
                    post_gain.to(DEV) if with_post else None, post_eps, pre_gain.to(DEV), pre_eps, packed, out[:m], n, epi)
    scale = float(ref.abs().max())
    assert float((out[:m].cpu().double() - ref).abs().max()) <= 8e-3 * scale
    assert torch.equal(h_dev.cpu(), h), "the rows that were read are not touched"
    if b is not None:
        assert float((h_out[:m].cpu().double() - hd).abs().max()) <= 2e-5 * float(hd.abs().max())
    else:
        assert float(h_out[:m].min()) == 7.0
    assert float(h_out[m].min()) == 7.0 and float(h_out[m].max()) == 7.0 and bool(torch.isnan(out[m].float()).all())


def test_product_of_one_token_refuses_what_it_cannot_do(G):
    assert not G.normed_ok(2, 4096, 2560, 0) and not G.normed_ok(1, 4096, 6152, 0) and not G.normed_ok(1, 4096, 2564, 0)
    assert not G.normed_ok(1, 262208, 2560, 0)            # (a workgroup would take more row blocks than its LDS holds sums for)
    k, n = 64, 32
    w = G.pack_weight(torch.zeros(n, k, dtype=torch.bfloat16, device=DEV))
    h = torch.zeros(1, k, device=DEV)
    gain = torch.ones(k, device=DEV)
    out = torch.empty(1, n, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError, match="of its own"):
        G.row_normed(h, h, torch.zeros(1, k, device=DEV), None, 0.0, gain, 1e-6, w, out, n)      # the sum in place
    with pytest.raises(ValueError):
        G.row_normed(torch.zeros(3, k, device=DEV), None, None, None, 0.0, gain, 1e-6, w, torch.empty(3, n, dtype=torch.bfloat16, device=DEV), n)
    with pytest.raises(ValueError):
        G.row_normed(h, None, None, None, 0.0, gain, 1e-6, w, out.float(), n)


def test_product_of_many_shapes(G):
    """Shapes drawn at random (fixed seed) across the kernels' cuts: tokens from 1 to 700, rows and
    columns that are multiples of nothing in particular (columns a multiple of 8, which the packed
    product requires), plain and sliced; each against a 64-bit product."""
    rng = np.random.default_rng(7)
    for case in range(48):
        m = int(rng.choice([1, 3, 8, 15, 16, 17, 31, 33, 48, 63, 64, 65, 100, 129, 255, 257, 400, 700]))
        n = int(rng.integers(1, 6000))
        k = 8 * int(rng.integers(1, 700))
        g = torch.Generator().manual_seed(case)
        x = torch.randn(m, k, generator=g).bfloat16()
        w = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
        packed = G.pack_weight(w.to(DEV))
        ref = x.double() @ w.double().T
        scale = float(ref.abs().max()) + 1e-6
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
        G.product(x.to(DEV), packed, out, n)
        assert float((out.cpu().double() - ref).abs().max()) <= 6e-3 * scale, (case, m, n, k)
        z = G.slices_for(m, n, k)
        if z > 1:
            parts = torch.full((z, m, n), float("nan"), device=DEV)
            G.skinny_slices(x.to(DEV), packed, parts, n)
            assert float((parts.cpu().double().sum(0) - ref).abs().max()) <= 2e-5 * scale * math.sqrt(k / 64), (case, m, n, k, z)


def test_gemm_skinny_refuses_what_it_cannot_do(G):
    w = G.pack_weight(torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV))
    out = torch.empty(65, 32, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(Exception, match="64"):
        G.skinny(torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV), w, out, 32)
    with pytest.raises(ValueError):
        G.skinny(torch.zeros(4, 60, dtype=torch.bfloat16, device=DEV), w, out[:4], 32)   # K no multiple of 8


@pytest.mark.parametrize("m,nh,hd,splits,n", [(8, 8, 256, 6, 2560), (1, 8, 256, 64, 2560), (16, 32, 128, 4, 5376),
                                              (3, 6, 64, 2, 100), (5, 16, 256, 3, 3840), (2, 4, 96, 9, 250),
                                              (13, 20, 128, 5, 72), (16, 8, 256, 11, 512), (1, 16, 256, 17, 3840)])
def test_product_of_the_decode_attention_s_partial_results(G, m, nh, hd, splits, n):
    """The output projection that merges the splits' partial results itself, against the merge
    written out (with its rows rounded to bfloat16, as the separate merge kernel leaves them) and an
    ordinary product.  Some splits are empty (reference -inf, sum 0), as behind a window's edge."""
    g = torch.Generator().manual_seed(m * 1000 + nh + splits)
    part_o = torch.randn(m, nh, splits, hd, generator=g)
    ref_m = torch.randn(m, nh, splits, generator=g) * 3
    sums = torch.rand(m, nh, splits, generator=g) * 30 + 0.5
    empty = torch.rand(m, nh, splits, generator=g) < 0.2
    empty[:, :, 0] = False                                   # every row keeps a split
    if m > 1:
        empty[1, 0, :] = True                                # but one: no key at all gives zeros
    ref_m[empty], sums[empty] = float("-inf"), 0.0
    part_o[empty] = 0.0
    part_ml = torch.stack([ref_m, sums], dim=-1).contiguous()
    runs = G.partials_runs(m, nh, hd, splits)
    assert 1 <= runs <= 8 and nh % runs == 0
    w = (torch.randn(n, nh * hd, generator=g) * 0.05).bfloat16()
    packed = G.pack_weight(w.to(DEV))
    out = torch.full((runs, m, n), float("nan"), device=DEV)
    G.product_of_partials(part_o.to(DEV), part_ml.to(DEV), packed, out, n)
    mx = ref_m.double().max(dim=-1, keepdim=True).values
    f = torch.where(torch.isinf(ref_m), torch.zeros_like(ref_m, dtype=torch.float64), torch.exp(ref_m.double() - mx))
    f = torch.nan_to_num(f, nan=0.0)
    l = (sums.double() * f).sum(-1)
    x = (part_o.double() * f[..., None]).sum(2) / torch.where(l > 0, l, torch.ones_like(l))[..., None]
    x = torch.where((l > 0)[..., None], x, torch.zeros_like(x)).reshape(m, nh * hd).bfloat16().double()
    ref = x @ w.double().T
    got = out.cpu().double()
    assert torch.isfinite(got).all()
    scale = float(ref.abs().max())
    # a merged value within rounding of a bfloat16 step's middle may round the other way: 2^-8 of one term
    assert float((got.sum(0) - ref).abs().max()) <= 3e-3 * scale
    # each slice is the product over its own run of heads
    cols = nh * hd // runs
    for r in range(runs):
        part = x[:, r * cols:(r + 1) * cols] @ w.double()[:, r * cols:(r + 1) * cols].T
        assert float((got[r] - part).abs().max()) <= 3e-3 * scale, r


def test_product_of_partial_results_refuses_what_it_cannot_do(G):
    assert G.partials_runs(17, 8, 256, 4) == 0          # more than one tile of tokens
    assert G.partials_runs(4, 8, 48, 4) == 0            # heads that are no whole k-steps of 32 columns
    assert G.partials_runs(4, 8, 256, 1) == 0           # nothing to merge
    assert G.partials_runs(16, 32, 128, 65) == 0        # more splits than the kernel merges
    with pytest.raises(ValueError, match="no kernel"):
        G.product_of_partials(torch.zeros(17, 8, 4, 256, device=DEV), torch.zeros(17, 8, 4, 2, device=DEV),
                              G.pack_weight(torch.zeros(32, 2048, dtype=torch.bfloat16, device=DEV)),
                              torch.zeros(8, 17, 32, device=DEV), 32)


# ---------------------------------------------------------------- matrix-core attention over packed pages
class _FakeStep:
    """What the attention op reads of a step."""

    def __init__(self, lens, queries_from, window):
        from agave_amd.parts import Workspace
        self.pos0 = [queries_from(L) for L in lens]
        self.n_new = [L - p for L, p in zip(lens, self.pos0)]
        self.n_seqs = len(lens)
        self.n_tokens = sum(self.n_new)
        self.max_new = max(self.n_new)
        cu = [0]
        for n in self.n_new:
            cu.append(cu[-1] + n)
        self.cu_dev = _i32(cu)
        self.tok_seq = _i32([b for b, n in enumerate(self.n_new) for _ in range(n)])
        self.tok_pos = _i32([p + i for p, n in zip(self.pos0, self.n_new) for i in range(n)])
        self.workspace = Workspace(torch.device(DEV))
        self.fixed_span = None

    @property
    def is_decode(self):
        return self.max_new == 1

    def page_span(self, window):
        span = 1
        for p0, n in zip(self.pos0, self.n_new):
            p = p0 + n - 1
            lo = max(0, p - window + 1) if window is not None else 0
            span = max(span, p // 64 - lo // 64 + 1)
        return span


def _mfma_attn_case(K, nh, nkv, hd, lens, window, scale, decode, seed=0, boost=None, last_row_only=False, fused=False):
    """Keys and values go into packed pages through the q/k kernel (no norm, no rotation); then
    either every position is a query (prefill) or only each sequence's last one (decode)."""
    from agave_amd.ops import attention_mfma
    g = torch.Generator().manual_seed(seed)
    hd_k = (hd + 31) // 32 * 32
    n_pages = sum((L + 63) // 64 for L in lens) + 2
    kp = torch.zeros(n_pages, nkv, 64, hd_k, dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros(n_pages, nkv, hd, 64, dtype=torch.bfloat16, device=DEV)
    perm = torch.randperm(n_pages, generator=g).tolist()
    width = max((L + 63) // 64 for L in lens)
    table = torch.full((len(lens), width), -1, dtype=torch.int32)
    ks, vs, qs = [], [], []
    for b, L in enumerate(lens):
        k = torch.randn(L, nkv, hd, generator=g).bfloat16()
        v = torch.randn(L, nkv, hd, generator=g).bfloat16()
        q = torch.randn(L, nh, hd, generator=g).bfloat16()
        if boost is not None:
            k = (k.float() - k.float().mean(dim=-1, keepdim=True)).bfloat16()
            k[boost] = 1.0
            q[L - 1] = 20.0 / (hd * scale)
        for i in range((L + 63) // 64):
            table[b, i] = perm.pop()
        ks.append(k); vs.append(v); qs.append(q)
    table, base = table.to(DEV), _i32([0] * len(lens))
    seq_all = _i32([b for b, L in enumerate(lens) for _ in range(L)])
    pos_all = _i32([i for L in lens for i in range(L)])
    k_all = torch.cat(ks).reshape(-1, nkv * hd).to(DEV)
    v_all = torch.cat(vs).reshape(-1, nkv * hd).to(DEV)
    K.qk_norm_rope_kv(None, k_all, v_all, None, None, None, 0.0, 0.0, None, 1.0, seq_all, pos_all, kp, vp, table, base,
                      0, nkv, hd, packed=True)
    step = _FakeStep(lens, (lambda L: L - 1) if decode else (lambda L: 0), window)
    q_sel = torch.cat([q[p0:] for q, p0 in zip(qs, step.pos0)]).reshape(-1, nh * hd).to(DEV)
    out = torch.full_like(q_sel, float("nan"))
    if fused:       # the decode kernel that also takes the new token's q and k: here it appends nothing
        attention_mfma.decode_fused(q_sel, None, None, out, None, None, 0.0, 0.0, None, 1.0, kp, vp, table, base, step,
                                    nh, nkv, hd, scale, window)
    else:
        attention_mfma.attention(q_sel, out, kp, vp, table, base, step, nh, nkv, hd, scale, window)
    if last_row_only and not decode:
        refs = []                                           # the caller checks rows of its choice
    elif last_row_only:
        refs = [_last_row_attention(q.double(), k.double(), v.double(), scale, window) for q, k, v in zip(qs, ks, vs)]
    else:
        refs = [P.attention_core(q.double(), k.double(), v.double(), scale, window)[p0:]
                for q, k, v, p0 in zip(qs, ks, vs, step.pos0)]
    return out.cpu().double().view(-1, nh, hd), (torch.cat(refs) if refs else (qs, ks)), vs


def _last_row_attention(q, k, v, scale, window):
    """The last position's attention alone, as a library softmax over its keys: what the whole
    table of scores would cost too much for at tens of thousands of keys.  q [L, nh, hd], k, v [L, nkv, hd]."""
    L, nh, _ = q.shape
    group = nh // k.shape[1]
    first = max(0, L - window) if window is not None else 0
    out = torch.empty(1, nh, v.shape[-1], dtype=torch.float64)
    for h in range(nh):
        scores = (k[first:, h // group] @ q[L - 1, h]) * scale
        out[0, h] = torch.softmax(scores, 0) @ v[first:, h // group]
    return out


@pytest.mark.parametrize("decode", [True, False])
@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 64, None), (6, 1, 16, 70), (3, 3, 48, 300), (8, 4, 256, 64),
                                              (2, 1, 128, None), (20, 1, 32, 129), (8, 2, 96, 1)])
def test_attn_mfma(K, decode, nh, nkv, hd, window):
    got, ref, _ = _mfma_attn_case(K, nh, nkv, hd, [1, 77, 300, 64, 65], window, 0.21 * (16 / hd) ** 0.5, decode)
    assert torch.isfinite(got).all()
    assert torch.allclose(got, ref, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("decode", [True, False])
def test_attn_mfma_long_sequences_split_over_workgroups(K, decode):
    from agave_amd.ops import attention_mfma
    assert attention_mfma.split_plan(40, 4)[0] > 1          # the decode launch below is split
    got, ref, _ = _mfma_attn_case(K, 4, 2, 128, [2500, 1031], None, 0.05, decode, seed=3)
    assert torch.allclose(got, ref, atol=2e-2, rtol=2e-2)
    got, ref, _ = _mfma_attn_case(K, 4, 2, 128, [2500, 1031], 1024, 0.05, decode, seed=4)
    assert torch.allclose(got, ref, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("nh,nkv,hd,lens,window", [(8, 4, 256, [20000, 9001, 100], None), (8, 4, 256, [20000, 9001], 1024),
                                                   (5, 1, 80, [33000], None), (2, 2, 64, [70000, 3], 4097)])
def test_attn_mfma_decode_over_tens_of_thousands_of_keys(K, nh, nkv, hd, lens, window):
    """Hundreds of pages a sequence, beside a short one: every share of the pages and their merge,
    with key 3 made to win in one pass (the furthest key there is) and random scores in the other."""
    g = torch.Generator().manual_seed(2)
    q, k, v = (torch.randn(9, n, 8, generator=g).double() for n in (4, 2, 2))
    for w in (None, 5):                                     # the helper is the plain function's last row
        assert torch.allclose(_last_row_attention(q, k, v, 0.3, w), P.attention_core(q, k, v, 0.3, w)[-1:], atol=1e-12)
    got, ref, _ = _mfma_attn_case(K, nh, nkv, hd, lens, window, 0.3 * (16 / hd) ** 0.5, True, seed=11, last_row_only=True)
    assert torch.isfinite(got).all()
    assert torch.allclose(got, ref, atol=2e-2, rtol=2e-2)
    if window is None:
        got, ref, vs = _mfma_attn_case(K, nh, nkv, hd, lens, None, 0.5, True, seed=12, boost=3, last_row_only=True)
        assert torch.allclose(got, ref, atol=2e-2, rtol=2e-2)
        assert torch.allclose(got[0, 0], vs[0][3, 0].double(), atol=2e-2)


@pytest.mark.parametrize("nh,nkv,hd,L,window", [(4, 2, 128, 20000, None), (8, 4, 256, 9001, 1024), (3, 1, 48, 40000, 5000)])
def test_attn_mfma_prefill_of_tens_of_thousands_of_tokens(K, nh, nkv, hd, L, window):
    """A prompt of hundreds of pages in one step; rows at the start, at page edges, in the middle
    and at the end are compared, each as the last row of the sequence that ends with it."""
    scale = 0.3 * (16 / hd) ** 0.5
    got, (qs, ks), vs = _mfma_attn_case(K, nh, nkv, hd, [L], window, scale, False, seed=13, last_row_only=True)
    assert torch.isfinite(got).all()
    for r in (0, 63, 64, 1023, 1024, L // 2 + 7, L - 65, L - 1):
        ref = _last_row_attention(qs[0][:r + 1].double(), ks[0][:r + 1].double(), vs[0][:r + 1].double(), scale, window)
        assert torch.allclose(got[r:r + 1], ref, atol=2e-2, rtol=2e-2), r


@pytest.mark.parametrize("nh,nkv,hd,lens,window", [(4, 2, 128, [1500], None), (4, 2, 128, [1500], 1024),
                                                   (8, 4, 256, [700, 300], None), (2, 2, 64, [1100, 64, 1], 600)])
def test_attn_mfma_prefill_blocks_shared_among_workgroups(K, nh, nkv, hd, lens, window):
    """A prompt with few blocks of positions: the blocks with a long reach are cut into pieces
    that go to workgroups of their own, and a second pass merges what they leave."""
    from agave_amd.ops import attention_mfma
    hw = 2 if nh // nkv >= 2 else 1
    plan = attention_mfma.plan_prefill_items([0] * len(lens), lens, window, (8 // hw) * 16, nkv, nh, hd)
    assert plan[2] > 1 and (plan[1] > 1).any() and (plan[1] == 1).any()      # some blocks in pieces, some whole
    got, ref, _ = _mfma_attn_case(K, nh, nkv, hd, lens, window, 0.3 * (16 / hd) ** 0.5, False, seed=7)
    assert torch.isfinite(got).all()
    assert torch.allclose(got, ref, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("how,hd", [(how, hd) for how in ("decode", "fused decode", "prefill") for hd in (32, 64, 128, 256)
                                    if not (how == "fused decode" and hd == 32)])      # (the fused kernel: 64, 128, 256)
def test_attn_mfma_far_key_and_window_edge(K, how, hd):
    """Key 3 of 700 is made to win every score of the last query; a window that ends just before
    it must lose it and one that just includes it must keep it.  Head size 32 takes the general
    kernels, 64 to 256 the fast ones (and the decode kernel that also handles the new token)."""
    kw = dict(decode=how != "prefill", fused=how == "fused decode", seed=1, boost=3)
    scale = 0.5 * (32 / hd) ** 0.5
    got, ref, vs = _mfma_attn_case(K, 2, 1, hd, [700], None, scale, **kw)
    assert torch.allclose(got[-1, 0], vs[0][3, 0].double(), atol=2e-2)
    got_w, _, _ = _mfma_attn_case(K, 2, 1, hd, [700], 696, scale, **kw)      # key 3 just outside
    assert not torch.allclose(got_w[-1, 0], vs[0][3, 0].double(), atol=1e-1)
    got_e, _, _ = _mfma_attn_case(K, 2, 1, hd, [700], 697, scale, **kw)      # just inside
    assert torch.allclose(got_e[-1, 0], vs[0][3, 0].double(), atol=2e-2)
    # the same at a window's edge that falls on a page's edge and one row either side of it
    for window, inside in ((700 - 64, False), (700 - 63, False), (700 - 3, True), (700 - 4, False)):
        got_p, _, _ = _mfma_attn_case(K, 2, 1, hd, [700], window, scale, **kw)
        assert torch.allclose(got_p[-1, 0], vs[0][3, 0].double(), atol=2e-2) == inside, window


# the last three shapes take the 128 x 128, 128 x 256 and 256 x 256 tiles, the others the 64 x 128 one; the
# shapes with few tiles and many columns are shared out along the columns (2, 5, 3 and 7 partial sums)
@pytest.mark.parametrize("m,n,k", [(65, 53, 72), (300, 256, 2560), (100, 250, 2560), (70, 200, 1560), (65, 2560, 10240),
                                   (257, 1000, 96), (2048, 300, 136), (130, 4100, 64),
                                   (1000, 4096, 96), (2048, 4090, 64), (1024, 10240, 72),
                                   # many stages (the loads run several stages ahead of the multiplications): each tile
                                   (300, 2000, 1000), (600, 5000, 1000), (1024, 5120, 1000), (1024, 10240, 1000),
                                   # 640 tiles: two rounds of 256 x 256 tiles and the last rows in tiles of half the height
                                   (2048, 20470, 64),
                                   # 320 tiles: one round and the last rows in tiles of a quarter of the size
                                   (1024, 20470, 64)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_gemm_tiled(G, m, n, k, out_dtype):
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
    packed = G.pack_weight(w.to(DEV))
    out = torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)
    G.product(x.to(DEV), packed, out, n)
    ref = x.double() @ w.double().T
    scale = float(ref.abs().max())
    tol = 2e-5 * scale * math.sqrt(k / 64) if out_dtype == torch.float32 else 6e-3 * scale
    assert float((out.cpu().double() - ref).abs().max()) <= tol


@pytest.mark.parametrize("m,n,k,slices", [
    (2048, 2560, 10240, 3),     # 160 tiles of 128 x 256: three slices, which run as 240 tiles of 256 x 256
    (4096, 2560, 10240, 1),     # 160 tiles of 256 x 256: one product
    (2000, 2552, 10248, 3),     # ragged edges
    (8192, 640, 10240, 3),      # 160 tiles of 128 x 256 whose slices in 256 x 256 would be 288: they stay 480 of 128 x 256
    (2048, 2560, 2048, 1),      # few columns: one product
    (1024, 2560, 10240, 3),     # a shorter prompt: 80 tiles of 128 x 256 in three slices
    (768, 2560, 10240, 4),      # 60 tiles in four
    (1024, 2560, 2048, 1),      # 80 tiles, but too few columns for a slice
    (300, 200, 4096, 8),        # next to no tiles of 64 x 128 (12): as many slices of those as leave eight stages each
    (256, 2560, 10240, 3),      # a short prompt: 80 tiles of 64 x 128 in three slices, one round of workgroups
    (384, 2560, 10240, 2),      # 120 tiles in two
    (130, 2560, 2048, 3),       # few columns: the slices keep six stages each (32 stages: five slices; 80 tiles: three)
    (100, 2560, 2048, 5),       # 40 tiles of 32 stages: five slices
    (256, 3840, 4096, 2),       # 120 tiles of 64 x 128 in two slices
    (384, 3840, 4096, 1),       # more tokens: 4,096 columns in slices of 128 x 256 tiles lose to the one product
    (200, 640, 320, 1)])        # five stages in all: one product
def test_gemm_tiled_in_slices(G, m, n, k, slices):
    """A product of many tokens whose tiles fill the compute units badly comes as 32-bit slices
    that add up to it, for a reader that adds them."""
    z = G.tiled_slices_for(m, n, k)
    assert z == slices
    if z == 1:
        return
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
    packed = G.pack_weight(w.to(DEV))
    out = torch.full((z, m, n), float("nan"), dtype=torch.float32, device=DEV)
    G.tiled_slices(x.to(DEV), packed, out, n)
    ref = x.to(DEV).double() @ w.to(DEV).double().T
    got = out.double().sum(0)
    assert float((got - ref).abs().max()) <= 2e-5 * float(ref.abs().max()) * math.sqrt(k / 64)
    assert float(out[0].abs().max()) > 0 and float(out[z - 1].abs().max()) > 0


@pytest.mark.parametrize("tile", [0, 1, 2, 3])
@pytest.mark.parametrize("m,n,k,z", [(300, 520, 1024, 1), (70, 200, 4096, 5), (513, 1000, 1544, 3), (256, 2560, 2048, 8)])
def test_gemm_tiled_every_tile_shape_in_slices(G, tile, m, n, k, z):
    """Each tile shape alone (256 x 256, 128 x 256, 128 x 128, 64 x 128), as one product and in
    slices, whatever the library's own choice for these sizes would be."""
    g = torch.Generator().manual_seed(m + n + k + tile)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
    packed = G.pack_weight(w.to(DEV))
    ref = x.double() @ w.double().T
    out = torch.full((z, m, n), float("nan"), dtype=torch.float32, device=DEV)
    G.tiled_slices_as(x.to(DEV), packed, out, n, tile)
    assert float((out.double().sum(0).cpu() - ref).abs().max()) <= 2e-5 * float(ref.abs().max()) * math.sqrt(k / 64)
    whole = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    G.tiled_as(x.to(DEV), packed, whole, n, tile)
    assert float((whole.double().cpu() - ref).abs().max()) <= 6e-3 * float(ref.abs().max())


@pytest.mark.parametrize("m,ff,k", [(70, 192, 64), (513, 1000, 96), (256, 20, 40), (1024, 5120, 1000), (2048, 10236, 64),
                                    (1024, 10236, 64)])
def test_gemm_tiled_geglu(G, m, ff, k):
    g = torch.Generator().manual_seed(ff + m)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(2 * ff, k, generator=g) * 0.2).bfloat16()
    packed = G.pack_weight(w.to(DEV), interleave_ff=ff)
    out = torch.full((m, ff), float("nan"), dtype=torch.bfloat16, device=DEV)
    G.product(x.to(DEV), packed, out, ff, epilogue=1)
    gu = x.double() @ w.double().T
    ref = P.gelu_tanh(gu[:, :ff]) * gu[:, ff:]
    assert float((out.cpu().double() - ref).abs().max()) <= 8e-3 * float(ref.abs().max())


def test_embedding_from_a_packed_table(G):
    table = (torch.randn(300, 72) * 0.05).bfloat16()
    packed = G.pack_weight(table.to(DEV))
    toks = [0, 299, 17, 17, 123, 16, 15]
    out = torch.empty(len(toks), 72, dtype=torch.float32, device=DEV)
    G.embed_scale_packed(_i32(toks), packed, math.sqrt(72.0), out, 300)
    assert torch.allclose(out.cpu().double(), P.embed(toks, table.double(), 72), atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("nh,nkv,hd,window,rot", [(8, 4, 256, 64, 128), (4, 2, 64, None, 16), (40, 2, 128, 1000, 64),
                                                  (2, 2, 128, None, 0)])
def test_attn_decode_fused_equals_the_two_kernels(K, nh, nkv, hd, window, rot):
    """The decode kernel that normalises, rotates and caches the new token itself must leave the
    same bits, in the output and in the cache pages, as the q/k kernel followed by the attention
    kernel; appending nothing (k None) must leave the pages alone."""
    from agave_amd.ops import attention as A
    g = torch.Generator().manual_seed(11)
    lens = [1, 64, 65, 300, 1500, 128]                  # positions at a page's first and last row among them
    B = len(lens)
    n_pages = sum((L + 63) // 64 for L in lens) + 1
    width = max((L + 63) // 64 for L in lens)
    perm = torch.randperm(n_pages, generator=g).tolist()
    table = torch.full((B, width), -1, dtype=torch.int32)
    for b, L in enumerate(lens):
        for i in range((L + 63) // 64):
            table[b, i] = perm.pop()
    table, base = table.to(DEV), _i32([0] * B)
    kp0 = torch.randn(n_pages, nkv, 64, hd, generator=g).bfloat16().to(DEV)      # older keys: any values
    vp0 = torch.randn(n_pages, nkv, hd, 64, generator=g).bfloat16().to(DEV)
    q = torch.randn(B, nh * hd, generator=g).bfloat16().to(DEV)
    k = torch.randn(B, nkv * hd, generator=g).bfloat16().to(DEV)
    v = torch.randn(B, nkv * hd, generator=g).bfloat16().to(DEV)
    qg = (1 + 0.2 * torch.randn(hd, generator=g)).to(DEV)
    kg = (1 + 0.2 * torch.randn(hd, generator=g)).to(DEV)
    inv_freq = torch.exp(-torch.arange(rot).float() / max(rot, 1) * 5).to(DEV) if rot else None
    step = _FakeStep(lens, lambda L: L - 1, window)
    scale = 0.3 * (16 / hd) ** 0.5
    outs = []
    for fused in (True, False):
        kp, vp = kp0.clone(), vp0.clone()
        out = torch.full_like(q, float("nan"))
        q_rot = torch.empty_like(q)
        if fused:
            A.qk_attention(q, k, v, q_rot, out, qg, kg, 1e-5, 2e-6, inv_freq, 0.5, kp, vp, table, base, step,
                           nh, nkv, hd, scale, window, True)
        else:
            K.qk_norm_rope_kv(q, k, v, q_rot, qg, kg, 1e-5, 2e-6, inv_freq, 0.5, step.tok_seq, step.tok_pos, kp, vp,
                              table, base, nh, nkv, hd, packed=True)
            A.attention(q_rot, out, kp, vp, table, base, step, nh, nkv, hd, scale, window, True)
        torch.cuda.synchronize()
        outs.append((out, kp, vp))
    assert torch.isfinite(outs[0][0].float()).all()
    for a, b, what in zip(outs[0], outs[1], ("output", "K pages", "V pages")):
        assert torch.equal(a, b), what
    # a run that appends nothing: queries only, pages untouched
    kp, vp = outs[1][1].clone(), outs[1][2].clone()
    out = torch.full_like(q, float("nan"))
    A.qk_attention(q, None, None, torch.empty_like(q), out, qg, kg, 1e-5, 2e-6, inv_freq, 0.5, kp, vp, table, base,
                   step, nh, nkv, hd, scale, window, True)
    assert torch.equal(out, outs[1][0]) and torch.equal(kp, outs[1][1]) and torch.equal(vp, outs[1][2])
