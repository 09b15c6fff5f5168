"""Every kernel entry point beside its plain C++ twin (rbitnet_amd/csrc/plain.cpp): the same
arguments, device tensors for the one and host tensors for the other, at sizes that fill no tile
and at the edges (one token, a page's last and first position, rows chosen by index, terms to be
added up).  The twins sum in double and round once, so the bounds here are the kernels' own
rounding: float32 results to 1e-5 of the largest value, bfloat16 results to one step of their
last bit."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
I32 = torch.int32
BF, F32 = torch.bfloat16, torch.float32


@pytest.fixture(scope="module")
def lib():
    from rbitnet_amd.csrc.lib import kernels
    return kernels()


@pytest.fixture(scope="module")
def twin():
    from rbitnet_amd.csrc.plain import plain_kernels
    return plain_kernels()


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _close(got, want, what=""):
    """got (device) against want (host): relative to the largest wanted magnitude."""
    g, w = got.detach().cpu().double(), want.double()
    assert g.shape == w.shape, (what, g.shape, w.shape)
    assert not torch.isnan(g).any(), what
    tol = 1e-5 if got.dtype == F32 else 8e-3
    err = float((g - w).abs().max() / w.abs().max().clamp_min(1e-30))
    assert err < tol, f"{what}: {err}"


def _both(lib, twin, name, host_args, outputs, **kw):
    """Calls lib.<name> on device copies and twin.<name> on the host tensors; returns
    {index of an output argument: (device result, host result)}."""
    dev_args = [a.to(DEV) if isinstance(a, torch.Tensor) else a for a in host_args]
    dev_kw = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in kw.items()}
    getattr(lib, name)(*dev_args, **dev_kw)
    getattr(twin, name)(*host_args, **kw)
    torch.cuda.synchronize()
    pick = lambda args, kws, i: kws[i] if isinstance(i, str) else args[i]
    return {i: (pick(dev_args, dev_kw, i), pick(host_args, kw, i)) for i in outputs}


@pytest.mark.parametrize("dtype", [F32, BF])
def test_embedding(lib, twin, dtype):
    g = _gen(1)
    for vocab, width, n in ((11, 7, 5), (300, 4096, 17)):
        table = torch.randn(vocab, width, generator=g).to(dtype)
        ids = torch.randint(0, vocab, (n,), generator=g).to(I32)
        ids[0], ids[-1] = vocab - 1, 0
        for dev, host in _both(lib, twin, "embed_gather", [table, ids, torch.empty(n, width)], [2]).values():
            assert torch.equal(dev.cpu(), host)


@pytest.mark.parametrize("out_dtype", [F32, BF])
@pytest.mark.parametrize("width", [33, 1000, 4096, 8192 + 16])
def test_add_rmsnorm(lib, twin, out_dtype, width):
    g = _gen(width)
    n = 5
    gain = 1 + 0.1 * torch.randn(width, generator=g)
    rows = torch.tensor([4, 0, 2], dtype=I32)
    for delta_shape in (None, (n, width), (3, n, width)):
        for chosen in (None, rows):
            x = torch.randn(n, width, generator=g)
            delta = None if delta_shape is None else torch.randn(*delta_shape, generator=g)
            out = torch.empty(n if chosen is None else 3, width, dtype=out_dtype)
            res = _both(lib, twin, "add_rmsnorm", [x, delta, gain, 1e-5, chosen, out], [0, 5])
            _close(*res[5], what=f"norm {delta_shape} {chosen is not None}")
            _close(*res[0], what="stream")              # updated in place, or left alone with chosen rows


@pytest.mark.parametrize("dtype", [F32, BF])
@pytest.mark.parametrize("style", [0, 1])
def test_rope_kv_write(lib, twin, dtype, style):
    g = _gen(10 + style)
    hq, hk, d = 6, 2, 24
    past, q_lens = [63, 0, 130], [3, 1, 2]
    tok_pos = torch.tensor([p + i for p, q in zip(past, q_lens) for i in range(q)], dtype=I32)
    tok_seq = torch.tensor([b for b, q in enumerate(q_lens) for _ in range(q)], dtype=I32)
    bt = torch.tensor([[5, 2, 0], [7, 0, 0], [1, 3, 6]], dtype=I32)
    n = int(tok_pos.numel())
    angles = torch.arange(200, dtype=torch.float64)[:, None] * (10000.0 ** (-2.0 * torch.arange(d // 2) / d))[None, :]
    cos, sin = torch.cos(angles).float(), torch.sin(angles).float()
    for terms in (1, 3):
        for tables in ((cos, sin), (None, None)):
            shape = (n, (hq + 2 * hk) * d) if terms == 1 else (terms, n, (hq + 2 * hk) * d)
            qkv = torch.randn(*shape, generator=g)
            args = [qkv, tables[0], tables[1], style, torch.empty(n, hq, d, dtype=dtype),
                    torch.zeros(8, hk, 64, d, dtype=dtype), torch.zeros(8, hk, 64, d, dtype=dtype), tok_pos, tok_seq, bt,
                    hq, hk, d]
            res = _both(lib, twin, "rope_kv_write", args, [4, 5, 6])
            for i in (4, 5, 6):
                _close(*res[i], what=f"rope output {i}, {terms} terms")
                if terms == 1:
                    assert torch.equal(res[i][0].cpu(), res[i][1])       # the same float32 operations: the same bits
    # a layer that keeps no cache: q only
    qkv = torch.randn(n, hq * d, generator=g)
    res = _both(lib, twin, "rope_kv_write", [qkv, cos, sin, style, torch.empty(n, hq, d, dtype=dtype), None, None,
                                             tok_pos, tok_seq, bt, hq, 0, d], [4])
    assert torch.equal(res[4][0].cpu(), res[4][1])


def test_swiglu(lib, twin):
    g = _gen(3)
    gu = torch.randn(7, 2 * 172, generator=g) * 4
    for dtype in (F32, BF):
        res = _both(lib, twin, "swiglu", [gu, torch.empty(7, 172, dtype=dtype)], [1])
        _close(*res[1], what="gate")


@pytest.mark.parametrize("m,n,k", [(1, 37, 50), (3, 256, 172), (16, 100, 64), (70, 96, 64), (200, 130, 48)])
def test_gemm_generic(lib, twin, m, n, k):
    g = _gen(m)
    for dtype in (F32, BF):
        a, w = torch.randn(m, k, generator=g).to(dtype), torch.randn(n, k, generator=g).to(dtype)
        res = _both(lib, twin, "gemm_generic", [a, w, torch.empty(m, n)], [2])
        _close(*res[2], what=f"generic product {dtype}")


@pytest.mark.parametrize("m", [1, 7, 16, 17, 33, 64])
@pytest.mark.parametrize("n,k", [(1000, 128), (4096, 512), (8208, 256), (160, 4096 + 128), (28672, 384), (16400, 256)])
def test_gemm_float32_of_few_tokens(lib, twin, m, n, k):
    """The float32 product for up to 64 tokens on the float32 MFMA (K a multiple of 128): row counts
    that fill no tile of 16, every number of token blocks, one and two row tiles a wave (two from 33 tokens
    and 16,384 rows on; 16,400 rows leave the last workgroup one), K in 1 to 4 waves with uneven shares, and
    the same product on the vector units."""
    g = _gen(m * 13 + n + k)
    a, w = torch.randn(m, k, generator=g), torch.randn(n, k, generator=g)
    res = _both(lib, twin, "gemm_generic", [a, w, torch.full((m, n), float("nan"))], [2])
    _close(*res[2], what="float32 product of few tokens")
    lib._lib.rb_tune_f32_few(0)
    try:
        other = torch.full((m, n), float("nan"), device=DEV)
        lib.gemm_generic(a.to(DEV), w.to(DEV), other)
    finally:
        lib._lib.rb_tune_f32_few(1)
    _close(other, res[2][1], what="float32 product of few tokens on the vector units")
    if n % 16 == 0:
        wf = torch.empty_like(w)
        twin.place_rows(w, wf, frag=True)
        frag = _both(lib, twin, "gemm_generic", [a, wf, torch.full((m, n), float("nan"))], [2], w_frag=True)
        _close(*frag[2], what="float32 product of few tokens, W fragment-major")
        assert torch.equal(frag[2][0], res[2][0])          # the same sums in the same order


@pytest.mark.parametrize("m,n,k", [(65, 992, 256), (200, 4096, 128), (300, 160, 1024)])
def test_gemm_float32_of_many_tokens_with_fragment_major_weights(lib, twin, m, n, k):
    """The float32 MFMA tiles reading W as rows and fragment-major: the same bits, and the twin's product."""
    g = _gen(m + n + k)
    a, w = torch.randn(m, k, generator=g), torch.randn(n, k, generator=g)
    wf = torch.empty_like(w)
    twin.place_rows(w, wf, frag=True)
    rows = _both(lib, twin, "gemm_generic", [a, w, torch.full((m, n), float("nan"))], [2])
    frag = _both(lib, twin, "gemm_generic", [a, wf, torch.full((m, n), float("nan"))], [2], w_frag=True)
    _close(*rows[2], what="float32 tiles, W as rows")
    _close(*frag[2], what="float32 tiles, W fragment-major")
    assert torch.equal(frag[2][0], rows[2][0]) and torch.equal(frag[2][1], rows[2][1])


@pytest.mark.parametrize("m", [1, 8, 16, 17, 64, 200, 600])
@pytest.mark.parametrize("n,k", [(992, 1024), (4096, 512), (1376, 200), (160, 4096)])
def test_gemm_bf16(lib, twin, m, n, k):
    """Every kernel the dispatcher picks for these sizes (skinny, tiled with and without K slices,
    the staged tiles for a K that is no multiple of 64), plain and gated, W as rows and fragment-major."""
    g = _gen(m * 7 + n)
    a = torch.randn(m, k, generator=g).to(BF)
    w = (torch.randn(n, k, generator=g) * 0.05).to(BF)
    for out_dtype in (F32, BF):
        res = _both(lib, twin, "gemm_bf16", [a, w, torch.empty(m, n, dtype=out_dtype)], [2])
        _close(*res[2], what="product")
    res = _both(lib, twin, "gemm_bf16", [a, w, torch.empty(m, n // 2, dtype=BF), 1], [2])
    _close(*res[2], what="gated product")
    if k % 64 == 0:
        wf = torch.empty_like(w)
        twin.place_rows(w, wf, frag=True)
        res = _both(lib, twin, "gemm_bf16", [a, wf, torch.empty(m, n)], [2], w_frag=True)
        _close(*res[2], what="fragment-major product")


@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("n,k", [(992, 1024), (12288, 512), (160, 4096 + 64)])
def test_gemm_bf16_few(lib, twin, m, n, k):
    g = _gen(m + n)
    a = torch.randn(m + 2, k, generator=g).to(BF)
    w = (torch.randn(n, k, generator=g) * 0.05).to(BF)
    rows = torch.randperm(m + 2, generator=g)[:m].to(I32)
    squares = torch.rand(m + 2, (k + 15) // 16, generator=g) * 16
    gain = 1 + 0.1 * torch.randn(n, generator=g)
    # prepared rows chosen by index, plain and gated
    res = _both(lib, twin, "gemm_bf16_few", [a, w, torch.empty(m, n)], [2], squares=squares, eps=1e-5, rows=rows)
    _close(*res[2], what="prepared rows")
    res = _both(lib, twin, "gemm_bf16_few", [a, w, torch.empty(m, n // 2, dtype=BF), 1], [2], squares=squares, eps=1e-5,
                rows=rows)
    _close(*res[2], what="prepared rows, gated")
    # the residual sum, and what it leaves for the norm that follows
    c = torch.randn(m, n, generator=g)
    res = _both(lib, twin, "gemm_bf16_few", [a[:m].contiguous(), w, c.clone(), 2], [2])
    _close(*res[2], what="C += product")
    res = _both(lib, twin, "gemm_bf16_few", [a[:m].contiguous(), w, c.clone(), 3], [2, "gained", "squares_out"], gain=gain,
                gained=torch.empty(m, n, dtype=BF), squares_out=torch.empty(m, (n + 15) // 16))
    _close(*res[2], what="C += product (3)")
    _close(*res["gained"], what="gained rows")
    _close(*res["squares_out"], what="sums of squares")


def _paged(g, past, q_lens, hk, d, dtype, n_pages=24):
    """A cache whose live positions hold random values and all others NaN, pages in random order."""
    total = [p + q for p, q in zip(past, q_lens)]
    width = max((t + 63) // 64 for t in total)
    perm = torch.randperm(n_pages, generator=g).tolist()
    bt = torch.zeros(len(past), width, dtype=I32)
    kp = torch.full((n_pages, hk, 64, d), float("nan"))
    vp = torch.full((n_pages, hk, 64, d), float("nan"))
    for b, t in enumerate(total):
        for j in range((t + 63) // 64):
            page = perm.pop()
            bt[b, j] = page
            live = min(64, t - 64 * j)
            kp[page, :, :live] = torch.randn(hk, live, d, generator=g)
            vp[page, :, :live] = torch.randn(hk, live, d, generator=g)
    tok_pos = torch.tensor([p + i for p, q in zip(past, q_lens) for i in range(q)], dtype=I32)
    tok_seq = torch.tensor([b for b, q in enumerate(q_lens) for _ in range(q)], dtype=I32)
    return kp.to(dtype), vp.to(dtype), bt, tok_pos, tok_seq


@pytest.mark.parametrize("dtype", [F32, BF])
@pytest.mark.parametrize("window", [0, 50])
@pytest.mark.parametrize("d", [24, 18, 128, 256])
def test_attention_generic(lib, twin, dtype, window, d):
    """Head sizes that are multiples of 4 (16-byte loads, the lanes in groups of 8, 32 and 64) and one that is
    not (the scalar kernel), which is also run on a size the other kernel takes."""
    g = _gen(20 + window + d)
    hq, hk = 6, 2
    past, q_lens = [63, 0, 130, 0], [3, 1, 70, 64]
    kp, vp, bt, tok_pos, tok_seq = _paged(g, past, q_lens, hk, d, dtype)
    n = int(tok_pos.numel())
    q = torch.randn(n, hq, d, generator=g).to(dtype)
    args = [q, kp, vp, torch.empty(n, hq * d, dtype=dtype), tok_pos, tok_seq, bt, hq, hk, d, d ** -0.5, window]
    res = _both(lib, twin, "attention_generic", args, [3])
    _close(*res[3], what="attention")
    # few tokens: 8 waves to a (token, head), which merge their states
    few = [a[-2:].contiguous() if isinstance(a, torch.Tensor) and a.shape[:1] == (n,) else a for a in args]
    res = _both(lib, twin, "attention_generic", few, [3])
    _close(*res[3], what="attention of two tokens")
    if d == 24:
        lib._lib.rb_tune_attention_vec(0)
        try:
            res = _both(lib, twin, "attention_generic", args, [3])
        finally:
            lib._lib.rb_tune_attention_vec(1)
        _close(*res[3], what="attention, scalar kernel")


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("hq,hk", [(8, 2), (4, 4), (6, 1)])
def test_attention_prefill_and_decode_bf16(lib, twin, d, hq, hk):
    g = _gen(d + hq)
    past, q_lens = [63, 0, 200, 0], [3, 1, 130, 64]
    kp, vp, bt, tok_pos, tok_seq = _paged(g, past, q_lens, hk, d, BF, n_pages=32)
    n = int(tok_pos.numel())
    q = torch.randn(n, hq, d, generator=g).to(BF)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=I32)
    for window in (0, 100):
        res = _both(lib, twin, "attention_prefill_bf16", [q, kp, vp, torch.empty(n, hq * d, dtype=BF), cu,
                                                          torch.tensor(past, dtype=I32), bt, len(past), max(q_lens), hq, hk,
                                                          d, d ** -0.5, window], [3])
        _close(*res[3], what=f"prefill attention, window {window}")
    # one token per sequence at its last position, in 1 and in 3 splits
    last = torch.tensor([p + ql - 1 for p, ql in zip(past, q_lens)], dtype=I32)
    qd = torch.randn(len(past), hq, d, generator=g).to(BF)
    for n_splits in (1, 3):
        ws = torch.empty(len(past) * hq * n_splits * (d + 2))
        res = _both(lib, twin, "attention_decode_bf16", [qd, kp, vp, torch.empty(len(past), hq * d, dtype=BF), last, bt, hq,
                                                         hk, d, d ** -0.5, 0, n_splits, ws], [3])
        _close(*res[3], what=f"decode attention, {n_splits} splits")
    # the fused form writes the new key and value at `last` itself
    angles = torch.arange(400, dtype=torch.float64)[:, None] * (10000.0 ** (-2.0 * torch.arange(d // 2) / d))[None, :]
    cos, sin = torch.cos(angles).float(), torch.sin(angles).float()
    qkv = torch.randn(2, len(past), (hq + 2 * hk) * d, generator=g)
    for style in (0, 1):
        ws = torch.empty(len(past) * hq * 2 * (d + 2))
        res = _both(lib, twin, "attention_decode_fused_bf16", [qkv, cos, sin, style, kp.clone(), vp.clone(),
                                                               torch.empty(len(past), hq * d, dtype=BF), last, bt, hq, hk,
                                                               d, d ** -0.5, 0, 2, ws], [4, 5, 6])
        _close(*res[6], what="fused decode attention")
        for i in (4, 5):
            dev, host = res[i]
            live = ~torch.isnan(host.float())
            assert torch.equal(torch.isnan(dev.cpu().float()), ~live)          # nothing but the new positions was written
            _close(torch.where(live.to(DEV), dev.float(), torch.zeros((), device=DEV)),
                   torch.where(live, host.float(), torch.zeros(())), what="cache after the fused step")


@pytest.mark.parametrize("vocab", [300, 4096, 128256])
def test_sample(lib, twin, vocab):
    g = _gen(vocab)
    n = 9
    logits = torch.randn(n, vocab, generator=g) * 4
    logits[0, 7] = logits[0, vocab - 1] = logits[0].max() + 1          # equal maxima
    logits[1, 3] = float("nan")
    res = _both(lib, twin, "sample", [logits, None, None, torch.empty(n, dtype=I32)], [3])
    assert torch.equal(res[3][0].cpu(), res[3][1])
    temps = torch.tensor([0.0, 0.7, 1.3, 0.2, 2.0, 1.0, 0.5, 0.9, 3.0])
    us = torch.tensor([0.3, 0.0, 0.999, 0.5, 0.25, 0.75, 0.1, 0.6, 0.45])
    res = _both(lib, twin, "sample", [logits, temps, us, torch.empty(n, dtype=I32)], [3])
    got, want = res[3][0].cpu(), res[3][1]
    for r in range(n):
        if int(got[r]) != int(want[r]):
            # sums in another order may move the choice by one place when u * total falls on a step of the running sum
            z = torch.nan_to_num(logits[r].double(), nan=-math.inf) / float(temps[r])
            cdf = torch.exp(z - z.max()).cumsum(0)
            gap = abs(float(cdf[int(got[r])] - cdf[int(want[r])])) / float(cdf[-1])
            assert abs(int(got[r]) - int(want[r])) == 1 and gap < 1e-6, (r, int(got[r]), int(want[r]))


def test_place_rows(lib, twin):
    g = _gen(5)
    src = torch.randn(48, 64, generator=g)
    for dtype in (F32, BF):
        for frag in (False, True):
            args = lambda row0, block, period: [src.to(dtype), torch.zeros(128, 64, dtype=dtype), row0, block, period]
            for a in (args(0, None, None), args(32, None, None), args(16, 16, 32)):
                res = _both(lib, twin, "place_rows", a, [1], frag=frag)
                assert torch.equal(res[1][0].cpu(), res[1][1])
