"""The decode attention's entry point that allocates nothing, called through ctypes: its output
against the existing entry point's (which takes the partial-result buffers from the caller) on
two calls in a row, the second with a smaller input, so that the array the library keeps holds
the first call's leftovers when the second runs."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float
SCRATCH_FLOATS = 2 << 20


def _i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


def _library():
    from agave_amd.ops import library
    lib = library.load("attention_mfma")
    lib.agave_attn_noalloc_init.argtypes = []
    lib.agave_attn_noalloc_init.restype = ctypes.c_int
    lib.agave_attn_decode_mfma_noalloc.argtypes = [_P, _L, _P, _L, _P, _P, _P, _I, _P, _I, _P, _P, _I, _I, _I, _I, _F, _I,
                                                   _I, _I, _I, _I, _P]
    lib.agave_attn_decode_mfma_noalloc.restype = ctypes.c_int
    lib.agave_attn_decode_mfma.argtypes = [_P, _L, _P, _L, _P, _P, _P, _P, _P, _I, _P, _I, _P, _P, _I, _I, _I, _I, _F, _I,
                                           _I, _I, _I, _I, _P]
    lib.agave_attn_decode_mfma.restype = ctypes.c_int
    lib.agave_last_error.restype = ctypes.c_char_p
    return lib


class Case:
    """Sequences of the given lengths in packed cache pages, and one query (the last position) each."""

    def __init__(self, lens, nh, nkv, hd, seed):
        from agave_amd.ops import kernels
        g = torch.Generator().manual_seed(seed)
        self.lens, self.nh, self.nkv, self.hd = lens, nh, nkv, hd
        n_pages = sum((L + 63) // 64 for L in lens) + 2
        self.kp = torch.zeros(n_pages, nkv, 64, (hd + 31) // 32 * 32, dtype=torch.bfloat16, device=DEV)
        self.vp = torch.zeros(n_pages, nkv, hd, 64, dtype=torch.bfloat16, device=DEV)
        perm = torch.randperm(n_pages, generator=g).tolist()
        self.width = max((L + 63) // 64 for L in lens)
        table = torch.full((len(lens), self.width), -1, dtype=torch.int32)
        for b, L in enumerate(lens):
            for i in range((L + 63) // 64):
                table[b, i] = perm.pop()
        self.table, self.base = table.to(DEV), _i32([0] * len(lens))
        k = torch.randn(sum(lens), nkv * hd, generator=g).bfloat16().to(DEV)
        v = torch.randn(sum(lens), nkv * hd, generator=g).bfloat16().to(DEV)
        self.k, self.v = k, v
        seq_all = _i32([b for b, L in enumerate(lens) for _ in range(L)])
        pos_all = _i32([i for L in lens for i in range(L)])
        kernels.qk_norm_rope_kv(None, k, v, None, None, None, 0.0, 0.0, None, 1.0, seq_all, pos_all, self.kp, self.vp,
                                self.table, self.base, 0, nkv, hd, packed=True)
        self.q = torch.randn(len(lens), nh * hd, generator=g).bfloat16().to(DEV)
        self.tok_seq = _i32(list(range(len(lens))))
        self.tok_pos = _i32([L - 1 for L in lens])
        self.n_pages = n_pages
        self.span = max((L + 63) // 64 for L in lens)

    def plan(self):
        """The engine's own plan for these sizes (the kernel for this head size shares half pages
        among the splits and looks at the number of splits only)."""
        from agave_amd.ops import attention_mfma
        chunks = -(-(self.nh // self.nkv) // 16)
        return attention_mfma.split_plan(self.span, len(self.lens) * self.nkv * chunks, self.hd)

    def scale(self):
        return 0.3 * (16 / self.hd) ** 0.5

    def plain(self):
        """softmax(q k^T * scale) v per sequence and head in float64, from the rows as they were given."""
        G, outs, at = self.nh // self.nkv, [], 0
        for b, L in enumerate(self.lens):
            k = self.k[at:at + L].double().cpu().view(L, self.nkv, self.hd)
            v = self.v[at:at + L].double().cpu().view(L, self.nkv, self.hd)
            q = self.q[b].double().cpu().view(self.nh, self.hd)
            rows = []
            for h in range(self.nh):
                w = torch.softmax(k[:, h // G] @ q[h] * self.scale(), 0)
                rows.append(w @ v[:, h // G])
            outs.append(torch.cat(rows))
            at += L
        return torch.stack(outs)

    def run(self, lib, noalloc: bool, splits=None, per=None):
        n = len(self.lens)
        if splits is None:
            splits, per = self.plan()
        out = torch.full_like(self.q, float("nan"))
        stream = torch.cuda.current_stream().cuda_stream
        tail = (self.kp.data_ptr(), self.vp.data_ptr(), self.table.data_ptr(), self.width, self.base.data_ptr(),
                self.n_pages, self.tok_seq.data_ptr(), self.tok_pos.data_ptr(), n, self.nh, self.nkv, self.hd,
                self.scale(), 0, splits, per, 1, 0, stream)
        if noalloc:
            rc = lib.agave_attn_decode_mfma_noalloc(self.q.data_ptr(), self.q.stride(0), out.data_ptr(), out.stride(0), *tail)
        else:
            part_o = torch.empty(n * self.nh * splits, self.hd, dtype=torch.float32, device=DEV)
            part_ml = torch.empty(n * self.nh * splits, 2, dtype=torch.float32, device=DEV)
            rc = lib.agave_attn_decode_mfma(self.q.data_ptr(), self.q.stride(0), out.data_ptr(), out.stride(0),
                                            part_o.data_ptr(), part_ml.data_ptr(), *tail)
            torch.cuda.synchronize()
        return rc, out


def test_two_calls_in_a_row_equal_the_entry_point_with_caller_buffers():
    lib = _library()
    assert lib.agave_attn_noalloc_init() == 0, lib.agave_last_error()
    big = Case([2500, 1031, 700], 8, 4, 256, seed=1)
    small = Case([300], 8, 4, 256, seed=2)
    assert big.plan()[0] > 1 and small.plan()[0] > 1          # both leave partial results in the library's array
    refs = []
    for case in (big, small):
        rc, ref = case.run(lib, noalloc=False)
        assert rc == 0, lib.agave_last_error()
        refs.append(ref)
        # the entry point it is compared with is itself right at these split counts
        assert torch.allclose(ref.double().cpu(), case.plain(), atol=2e-2, rtol=2e-2)
    # the two calls follow each other on one stream with nothing between them
    rc1, out1 = big.run(lib, noalloc=True)
    rc2, out2 = small.run(lib, noalloc=True)
    torch.cuda.synchronize()
    assert rc1 == 0 and rc2 == 0, lib.agave_last_error()
    for out, ref, what in ((out1, refs[0], "first call"), (out2, refs[1], "second, smaller call")):
        assert torch.isfinite(out.float()).all(), what
        assert torch.equal(out, ref), what
    # and once more the large one after the small one
    rc3, out3 = big.run(lib, noalloc=True)
    torch.cuda.synchronize()
    assert rc3 == 0 and torch.equal(out3, refs[0])
    # a batch of one at the engine's twelve splits
    single = Case([1500], 8, 4, 256, seed=5)
    assert single.plan()[0] == 12
    rc, out = single.run(lib, noalloc=True)
    torch.cuda.synchronize()
    assert rc == 0 and torch.allclose(out.double().cpu(), single.plain(), atol=2e-2, rtol=2e-2)
    # one share a sequence: nothing of the array is used
    rc, whole = small.run(lib, noalloc=True, splits=1, per=small.span)
    torch.cuda.synchronize()
    assert rc == 0 and torch.allclose(whole.float(), refs[1].float(), atol=2e-2, rtol=2e-2)


def test_a_step_beyond_the_array_is_refused_with_a_message():
    lib = _library()
    case = Case([200, 130], 8, 4, 256, seed=3)
    # 2 tokens x 8 heads x splits x 258 floats: 1100 splits would need 4.5 million floats
    splits = SCRATCH_FLOATS // (2 * 8 * 258) + 1
    rc, _ = case.run(lib, noalloc=True, splits=splits, per=1)
    assert rc != 0
    msg = lib.agave_last_error().decode()
    assert "exceed" in msg and str(SCRATCH_FLOATS) in msg
