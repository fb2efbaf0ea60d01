"""Each part of a layer alone against the plain implementation's function for it: the norm, the
position encoding, the attention mixer, the feed-forward and the two block arrangements, built
from their specs with sizes that no model of the other tests has."""
import math

import pytest
import torch

import plain_gemma3 as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


# ---------------------------------------------------------------- a step without a model
class Bench:
    """Workspace, cache and planner for one mixer's needs: what a part sees of the engine."""

    def __init__(self, dtype, kv_need=None, state_need=None, max_slots=4, max_context=256):
        from agave_amd.cache import KVCache
        from agave_amd.engine.step import StepPlanner
        from agave_amd.parts import BuildEnv, Workspace
        self.dtype = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
        self.ws = Workspace(torch.device(DEV))
        self.env = BuildEnv(self.dtype, torch.device(DEV), self.ws)
        kv = {0: kv_need} if kv_need is not None else {}
        st = {0: state_need} if state_need is not None else {}
        pages = {kv_need: max_slots * (max_context // 64)} if kv_need is not None else {}
        self.cache = KVCache(kv, st, max_slots, pages, self.dtype, torch.device(DEV), max_context)
        self.planner = StepPlanner(self.cache, 10, torch.device(DEV), self.ws)

    def step(self, slots, n_new):
        s = self.planner.plan(slots, [[0] * n for n in n_new], "none")
        return s

    def commit(self, s):
        self.planner.commit(s)


def weights_of(tensors, needs, dtype):
    from agave_amd.weights.loader import DictWeightSource
    t = {k: v.to(torch.bfloat16 if dtype == "bfloat16" else torch.float32) for k, v in tensors.items()}
    return DictWeightSource(t, needs)


def rnd(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).bfloat16().double()     # exactly representable in bfloat16


def check(got, ref, dtype, what):
    got, ref = got.double().cpu(), ref.double()
    scale = float(ref.abs().max())
    err = float((got - ref).abs().max())
    tol = 2e-5 if dtype == "float32" else 2e-2
    assert err <= tol * scale, f"{what} ({dtype}): error {err:.3e} against values up to {scale:.3e}"


DTYPES = ["float32", "bfloat16"]


# ---------------------------------------------------------------- norm
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("add_one", [True, False])
def test_rmsnorm_part(dtype, add_one):
    from agave_amd.config.spec import NormSpec
    from agave_amd.ops import kernels
    from agave_amd.parts import RmsNorm
    size, eps = 208, 3e-4
    spec = NormSpec("rmsnorm", size, eps, "n.weight", add_one)
    w = rnd((size,), 1, 0.3)
    b = Bench(dtype)
    part = RmsNorm(spec, weights_of({"n.weight": w}, RmsNorm.tensor_needs(spec), dtype), b.env)
    assert [(n.name, tuple(n.shape)) for n in RmsNorm.tensor_needs(spec)] == [("n.weight", (size,))]
    h = rnd((7, size), 2, 3.0)
    hd = h.float().to(DEV)
    out = torch.empty((7, size), dtype=b.dtype, device=DEV)
    kernels.residual_norm(hd, None, None, 0.0, out, part.gain, part.eps)
    check(out, P.rms_norm(h, w, eps, add_one), dtype, "norm")
    assert torch.equal(hd.cpu().double(), h)               # no branch: the residual stream is untouched


# ---------------------------------------------------------------- attention (with its position encoding)
def attention_spec(hidden, nh, nkv, hd, window, theta, factor, norms, eps=2e-5, position="rope", scale=None):
    from agave_amd.config.spec import AttentionSpec, NormSpec, PositionSpec
    pos = PositionSpec("rope", hd, theta, factor) if position == "rope" else PositionSpec(position)
    return AttentionSpec(
        kind="attention", hidden=hidden, n_heads=nh, n_kv_heads=nkv, head_dim=hd,
        scale=scale if scale is not None else 1.0 / math.sqrt(hd), window=window, position=pos,
        q_norm=NormSpec("rmsnorm", hd, eps, "a.qn", True) if norms else None,
        k_norm=NormSpec("rmsnorm", hd, eps, "a.kn", True) if norms else None,
        q_proj="a.q", k_proj="a.k", v_proj="a.v", o_proj="a.o")


def attention_on_bench(spec, t, dtype):
    """The attention part on a bench whose cache holds what the part says it needs."""
    from agave_amd.cache import GroupKey
    from agave_amd.parts import Attention
    b = Bench(dtype, GroupKey(spec.window, spec.n_kv_heads, spec.head_dim))
    part = Attention(spec, weights_of(t, Attention.tensor_needs(spec), dtype), b.env)
    assert part.kv_need() == b.cache.group_keys[0] and part.state_need() is None
    return b, part


def attention_tensors(spec, seed):
    qd, kvd = spec.n_heads * spec.head_dim, spec.n_kv_heads * spec.head_dim
    t = {"a.q": rnd((qd, spec.hidden), seed, 0.08), "a.k": rnd((kvd, spec.hidden), seed + 1, 0.08),
         "a.v": rnd((kvd, spec.hidden), seed + 2, 0.08), "a.o": rnd((spec.hidden, qd), seed + 3, 0.08)}
    if spec.q_norm is not None:
        t["a.qn"] = rnd((spec.head_dim,), seed + 4, 0.2)
        t["a.kn"] = rnd((spec.head_dim,), seed + 5, 0.2)
    return t


def plain_attention(spec, t, x):
    """The plain functions put together for one whole sequence x [T, hidden]."""
    T = x.shape[0]
    q = (x @ t["a.q"].T).view(T, spec.n_heads, spec.head_dim)
    k = (x @ t["a.k"].T).view(T, spec.n_kv_heads, spec.head_dim)
    v = (x @ t["a.v"].T).view(T, spec.n_kv_heads, spec.head_dim)
    if spec.q_norm is not None:
        q = P.rms_norm(q, t["a.qn"], spec.q_norm.eps)
        k = P.rms_norm(k, t["a.kn"], spec.k_norm.eps)
    if spec.position.kind == "rope":
        ang = P.rope_angles(torch.arange(T, dtype=torch.float64), spec.position.rotary_dim, spec.position.theta,
                            spec.position.factor)
        q, k = P.apply_rope(q, ang), P.apply_rope(k, ang)
    o = P.attention_core(q, k, v, spec.scale, spec.window)
    return o.reshape(T, -1) @ t["a.o"].T


def run_mixer_ragged(b, part, xs, first):
    """The sequences' first ``first[i]`` rows in one step, then one row each per step until every
    sequence is used up (shorter ones leave).  Returns the outputs per sequence."""
    slots = [b.cache.alloc_slot() for _ in xs]
    outs = [[] for _ in xs]

    def run(idx, chunks):
        st = b.step([slots[i] for i in idx], [c.shape[0] for c in chunks])
        x = torch.cat(chunks, 0).to(b.dtype).to(DEV)
        y = part.forward(x, st, 0, True).float().cpu()
        b.commit(st)
        o = 0
        for i, c in zip(idx, chunks):
            outs[i].append(y[o:o + c.shape[0]].clone())
            o += c.shape[0]

    run(list(range(len(xs))), [x[:f] for x, f in zip(xs, first)])
    done = list(first)
    while True:
        idx = [i for i, x in enumerate(xs) if done[i] < x.shape[0]]
        if not idx:
            break
        run(idx, [xs[i][done[i]:done[i] + 1] for i in idx])
        for i in idx:
            done[i] += 1
    for s in slots:
        b.cache.free_slot(s)
    return [torch.cat(o, 0) for o in outs]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", ["window_gqa", "global_scaled", "bare_mha"])
def test_attention_part(dtype, case):
    if case == "window_gqa":       # window smaller than a page edge away, 3 query heads per kv head
        spec = attention_spec(112, 6, 2, 48, 37, 5000.0, 1.0, True)
        lens, first = (90, 41, 67), (70, 41, 3)
    elif case == "global_scaled":  # linear position scaling, another eps and scale
        spec = attention_spec(96, 4, 4, 32, None, 123456.0, 4.0, True, eps=1e-3, scale=0.21)
        lens, first = (130, 20), (100, 1)
    else:                          # no q/k norm and no position encoding: plain softmax attention
        spec = attention_spec(80, 5, 5, 16, None, 0.0, 1.0, False, position="none")
        lens, first = (66, 9), (64, 5)
    t = attention_tensors(spec, 10)
    b, part = attention_on_bench(spec, t, dtype)
    xs = [rnd((n, spec.hidden), 20 + i) for i, n in enumerate(lens)]
    outs = run_mixer_ragged(b, part, xs, first)
    for i, (x, o) in enumerate(zip(xs, outs)):
        check(o, plain_attention(spec, t, x), dtype, f"{case} sequence {i}")
    assert b.cache.slots.n_free == b.cache.max_slots


@pytest.mark.parametrize("dtype", DTYPES)
def test_bare_attention_equals_library_softmax(dtype):
    """Without norm, rotation, mask or grouping a single query row is softmax(q K^T s) V, which a
    library routine states independently of the plain implementation."""
    spec = attention_spec(64, 2, 2, 32, None, 0.0, 1.0, False, position="none", scale=0.3)
    t = attention_tensors(spec, 40)
    b, part = attention_on_bench(spec, t, dtype)
    x = rnd((50, 64), 41)
    out = run_mixer_ragged(b, part, [x], (50,))[0]
    q = (x @ t["a.q"].T).view(50, 2, 32).transpose(0, 1)
    k = (x @ t["a.k"].T).view(50, 2, 32).transpose(0, 1)
    v = (x @ t["a.v"].T).view(50, 2, 32).transpose(0, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=0.3)
    check(out, ref.transpose(0, 1).reshape(50, 64) @ t["a.o"].T, dtype, "bare attention")


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotation_depends_on_distance_only(dtype):
    """With rotation and no norm the scores depend on the distance of query and key only.  The
    same rows run once from position 0 and once behind 29 other positions of the slot; a window
    of 12 keeps those out of reach, so rows from the 12th on see the same keys at the same
    distances and must give the same output."""
    spec = attention_spec(64, 2, 1, 32, 12, 777.0, 1.0, False)
    t = attention_tensors(spec, 50)
    b, part = attention_on_bench(spec, t, dtype)
    x = rnd((40, 64), 51)
    at_zero = run_mixer_ragged(b, part, [x], (40,))[0]
    shifted = run_mixer_ragged(b, part, [torch.cat([rnd((29, 64), 52), x], 0)], (69,))[0][29:]
    check(shifted[11:], at_zero[11:], dtype, "shifted positions")
    # and the rotation is really applied: without it the result differs
    nspec = attention_spec(64, 2, 1, 32, 12, 0.0, 1.0, False, position="none")
    nb, npart = attention_on_bench(nspec, t, dtype)
    no_rot = run_mixer_ragged(nb, npart, [x], (40,))[0]
    assert float((no_rot[11:] - at_zero[11:]).abs().max()) > 1e-3 * float(at_zero.abs().max())


# ---------------------------------------------------------------- feed-forward
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,inter,rows", [(112, 200, 5), (96, 72, 70)])
def test_gated_ffn_part(dtype, hidden, inter, rows):
    from agave_amd.config.spec import GatedFfnSpec
    from agave_amd.parts import GatedFfn
    spec = GatedFfnSpec(kind="gated_dense", hidden=hidden, intermediate=inter, activation="gelu_tanh",
                        gate_proj="f.g", up_proj="f.u", down_proj="f.d")
    t = {"f.g": rnd((inter, hidden), 60, 0.1), "f.u": rnd((inter, hidden), 61, 0.1), "f.d": rnd((hidden, inter), 62, 0.1)}
    b = Bench(dtype)
    part = GatedFfn(spec, weights_of(t, GatedFfn.tensor_needs(spec), dtype), b.env)
    x = rnd((rows, hidden), 63, 2.0)
    y = part.forward(x.to(b.dtype).to(DEV), None)
    check(y, P.geglu(x, t["f.g"], t["f.u"], t["f.d"]), dtype, "feed-forward")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("activation", ["silu", "gelu", "relu"])
@pytest.mark.parametrize("rows", [6, 150])
def test_gated_ffn_part_with_another_activation(dtype, activation, rows):
    """The activation is the spec's: with another one than the tanh form of GELU the stacked
    gate/up product keeps its rows in order and the elementwise kernel applies the activation,
    for a handful of tokens (skinny product) and for a prompt's worth (tiled product)."""
    from agave_amd.config.spec import GatedFfnSpec
    from agave_amd.parts import GatedFfn
    hidden, inter = 96, 200
    spec = GatedFfnSpec(kind="gated_dense", hidden=hidden, intermediate=inter, activation=activation,
                        gate_proj="f.g", up_proj="f.u", down_proj="f.d")
    t = {"f.g": rnd((inter, hidden), 70, 0.1), "f.u": rnd((inter, hidden), 71, 0.1), "f.d": rnd((hidden, inter), 72, 0.1)}
    b = Bench(dtype)
    part = GatedFfn(spec, weights_of(t, GatedFfn.tensor_needs(spec), dtype), b.env)
    assert not part.gate_up.interleave_ff
    x = rnd((rows, hidden), 73, 2.0)
    y = part.forward(x.to(b.dtype).to(DEV), None)
    y = y.sum(0) if y.dim() == 3 else y
    act = {"silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu, "relu": torch.relu}[activation]
    xd = x.to(b.dtype).double()
    ref = (act(xd @ t["f.g"].double().T) * (xd @ t["f.u"].double().T)) @ t["f.d"].double().T
    check(y, ref, dtype, f"feed-forward with {activation}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,out_f,in_f,slices_ok", [(5, 96, 200, False), (8, 2560, 10240, True), (256, 3840, 4096, True),
                                                     (150, 130, 72, True)])
def test_linear_with_a_bias_on_every_path(dtype, rows, out_f, in_f, slices_ok):
    """y = W x + b with two stacked matrices of which one has a bias: as one tensor and as 32-bit
    slices that add up (few rows of a long product, and a prompt's worth of rows), the bias
    being added once, not once a slice."""
    from agave_amd.parts import Linear
    b = Bench(dtype)
    top = out_f // 3
    w0, w1 = rnd((top, in_f), 80, 0.05), rnd((out_f - top, in_f), 81, 0.05)
    bias1 = rnd((out_f - top,), 82, 2.0)
    tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    lin = Linear([w0.to(tdt), w1.to(tdt)], b.env, "biased", biases=[None, bias1.to(tdt)])
    assert lin.bias.dtype == torch.float32 and float(lin.bias[:top].abs().max()) == 0.0
    x = rnd((rows, in_f), 83, 1.0)
    y = lin.forward(x.to(b.dtype).to(DEV), slices_ok=slices_ok)
    if dtype == "bfloat16" and (rows, out_f, in_f) in ((8, 2560, 10240), (256, 3840, 4096)):
        assert y.dim() == 3 and y.shape[0] > 1, "this shape was chosen because it comes in slices"
    y = y.sum(0) if y.dim() == 3 else y
    ref = x @ torch.cat([w0, w1]).T + torch.cat([torch.zeros(top, dtype=torch.float64), bias1])
    check(y, ref, dtype, "linear with a bias")
    with pytest.raises(ValueError, match="bias of shape"):
        Linear([w0.to(tdt)], b.env, "wrong", biases=[bias1.to(tdt)[:top + 1]])


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_ffn_part_with_biases(dtype):
    """Biases on gate, up and down: the gate/up product then keeps its rows in order (the product
    that ends in the activation has no place for a bias) and the elementwise kernel follows."""
    from agave_amd.config.spec import GatedFfnSpec
    from agave_amd.parts import GatedFfn
    hidden, inter = 96, 200
    spec = GatedFfnSpec(kind="gated_dense", hidden=hidden, intermediate=inter, activation="gelu_tanh",
                        gate_proj="f.g", up_proj="f.u", down_proj="f.d", gate_bias="f.gb", up_bias="f.ub", down_bias="f.db")
    t = {"f.g": rnd((inter, hidden), 70, 0.1), "f.u": rnd((inter, hidden), 71, 0.1), "f.d": rnd((hidden, inter), 72, 0.1),
         "f.gb": rnd((inter,), 74, 1.0), "f.ub": rnd((inter,), 75, 1.0), "f.db": rnd((hidden,), 76, 1.0)}
    b = Bench(dtype)
    needs = GatedFfn.tensor_needs(spec)
    assert {n.name for n in needs} == set(t)
    part = GatedFfn(spec, weights_of(t, needs, dtype), b.env)
    assert not part.gate_up.interleave_ff
    for rows in (6, 150):
        x = rnd((rows, hidden), 73, 2.0)
        y = part.forward(x.to(b.dtype).to(DEV), None)
        y = y.sum(0) if y.dim() == 3 else y
        xd = x.to(b.dtype).double()
        ref = (P.gelu_tanh(xd @ t["f.g"].T + t["f.gb"]) * (xd @ t["f.u"].T + t["f.ub"])) @ t["f.d"].T + t["f.db"]
        check(y, ref, dtype, f"feed-forward with biases, {rows} rows")


def test_gated_ffn_at_a_prompts_length_comes_in_slices_that_the_residual_kernel_adds():
    """The benchmark model's feed-forward at 2,048 tokens: the down product's tiles would leave
    many compute units idle, so it comes as 32-bit slices; summed, and added to the residual
    stream by the norm kernel, they give what the formula gives (the plain formula runs on the
    GPU here, in 64-bit: it is a hundred GFLOP)."""
    from agave_amd.config.spec import GatedFfnSpec, NormSpec
    from agave_amd.parts import GatedFfn, add_pending_and_norm, lookup
    hidden, inter, rows = 2560, 10240, 2048
    spec = GatedFfnSpec(kind="gated_dense", hidden=hidden, intermediate=inter, activation="gelu_tanh",
                        gate_proj="f.g", up_proj="f.u", down_proj="f.d")
    t = {"f.g": rnd((inter, hidden), 60, 0.02), "f.u": rnd((inter, hidden), 61, 0.02), "f.d": rnd((hidden, inter), 62, 0.02)}
    b = Bench("bfloat16")
    part = GatedFfn(spec, weights_of(t, GatedFfn.tensor_needs(spec), "bfloat16"), b.env)
    x = rnd((rows, hidden), 63, 1.0)
    y = part.forward(x.to(torch.bfloat16).to(DEV), None)
    assert y.dim() == 3 and y.shape[0] > 1 and y.dtype == torch.float32
    ref = P.geglu(x.to(DEV), t["f.g"].to(DEV), t["f.u"].to(DEV), t["f.d"].to(DEV)).cpu()
    check(y.sum(0), ref, "bfloat16", "feed-forward in slices")
    # the norm kernel adds the slices to the residual stream and normalises the sum
    nspec = NormSpec("rmsnorm", hidden, 1e-6, "n.w", True)
    norm = lookup("norm", "rmsnorm")(nspec, weights_of({"n.w": rnd((hidden,), 64, 0.1)}, lookup("norm", "rmsnorm").tensor_needs(nspec),
                                                        "bfloat16"), b.env)
    h0 = rnd((rows, hidden), 65, 1.0).float()
    h = h0.clone().to(DEV)
    out = torch.empty(rows, hidden, dtype=torch.bfloat16, device=DEV)
    add_pending_and_norm(h, (y, None), norm, out)
    want_h = h0.double() + ref
    check(h, want_h, "bfloat16", "residual stream after the slices")
    check(out, P.rms_norm(want_h, rnd((hidden,), 64, 0.1), 1e-6, add_one=True), "bfloat16", "norm of the sum")


def test_gated_ffn_refuses_unknown_activation():
    from agave_amd.config.spec import GatedFfnSpec
    from agave_amd.parts import GatedFfn
    spec = GatedFfnSpec(kind="gated_dense", hidden=32, intermediate=32, activation="swish_of_tomorrow",
                        gate_proj="g", up_proj="u", down_proj="d")
    with pytest.raises(ValueError, match="activation"):
        GatedFfn(spec, None, Bench("float32").env)


# ---------------------------------------------------------------- blocks
def block_spec(kind, hidden, inter, window):
    from agave_amd.config.spec import GatedFfnSpec, LayerSpec, NormSpec
    att = attention_spec(hidden, 4, 2, 32, window, 9000.0, 1.0, True)
    ffn = GatedFfnSpec(kind="gated_dense", hidden=hidden, intermediate=inter, activation="gelu_tanh",
                       gate_proj="f.g", up_proj="f.u", down_proj="f.d")

    def n(name):
        return NormSpec("rmsnorm", hidden, 1e-5, name, True)
    return LayerSpec(kind=kind, mixer=att, ffn=ffn, pre_mixer_norm=n("n.0"), post_mixer_norm=n("n.1"),
                     pre_ffn_norm=n("n.2"), post_ffn_norm=n("n.3"))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["sandwich", "prenorm"])
def test_block_part(dtype, kind):
    """A block returns its last branch as pending; adding it with its post norm gives the
    residual stream that the formula gives."""
    from agave_amd.parts import add_pending_and_norm, lookup
    hidden, inter = 96, 136
    spec = block_spec(kind, hidden, inter, 50)
    cls = lookup("block", kind)
    t = attention_tensors(spec.mixer, 70)
    t.update({"f.g": rnd((inter, hidden), 80, 0.1), "f.u": rnd((inter, hidden), 81, 0.1), "f.d": rnd((hidden, inter), 82, 0.1)})
    for i in range(4):
        t[f"n.{i}"] = rnd((hidden,), 90 + i, 0.2)
    needs = cls.tensor_needs(spec)
    names = {n.name for n in needs}
    if kind == "prenorm":
        assert "n.1" not in names and "n.3" not in names
        t = {k: v for k, v in t.items() if k in names}
    from agave_amd.cache import GroupKey
    b = Bench(dtype, GroupKey(spec.mixer.window, spec.mixer.n_kv_heads, spec.mixer.head_dim))
    block = cls(spec, weights_of(t, needs, dtype), b.env)
    assert block.mixer.kv_need() == b.cache.group_keys[0]

    T = 75
    h0 = rnd((T, hidden), 99, 1.5)
    slot = b.cache.alloc_slot()
    h = h0.float().to(DEV)
    st = b.step([slot], [T])
    pending = block.forward(h, None, st, 0, True)
    b.commit(st)
    out = torch.empty((T, hidden), dtype=b.dtype, device=DEV)
    final_gain = rnd((hidden,), 100, 0.2)

    from agave_amd.config.spec import NormSpec
    final_spec = NormSpec("rmsnorm", hidden, 1e-5, "final", True)
    final_needs = lookup("norm", "rmsnorm").tensor_needs(final_spec)
    final = lookup("norm", "rmsnorm")(final_spec, weights_of({"final": final_gain}, final_needs, dtype), b.env)
    add_pending_and_norm(h, pending, final, out)

    a = plain_attention(spec.mixer, t, P.rms_norm(h0, t["n.0"], 1e-5))
    r = h0 + (P.rms_norm(a, t["n.1"], 1e-5) if kind == "sandwich" else a)
    f = P.geglu(P.rms_norm(r, t["n.2"], 1e-5), t["f.g"], t["f.u"], t["f.d"])
    r = r + (P.rms_norm(f, t["n.3"], 1e-5) if kind == "sandwich" else f)
    check(h, r, dtype, f"{kind} residual stream")
    check(out, P.rms_norm(r, final_gain, 1e-5), dtype, f"{kind} norm after the block")
    assert h.dtype == torch.float32
