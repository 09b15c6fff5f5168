"""Each HIP kernel alone against a plain float32 (or float64) computation in torch, at
sizes other than the engine tests use: widths that are no power of two, head sizes in
steps of 16, odd head groups, rows that do not fill a tile."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def lib():
    from rbitnet_amd.csrc.lib import kernels
    return kernels()


def _rel(got, want):
    want = want.double()
    return float((got.double().cpu() - want.cpu()).abs().max() / want.abs().max().clamp_min(1e-30))


# ------------------------------------------------------------------------ linear
def test_reference_matvec_vectors(lib):
    """The reference's own vectors: kernels.rs:35-40 and tests/golden_kernels.rs:12-18."""
    w = torch.tensor([[1., 0.], [-1., 1.]], device=DEV)
    x = torch.tensor([[2., 3.]], device=DEV)
    c = torch.empty(1, 2, device=DEV)
    lib.gemm_generic(x, w, c)
    assert torch.allclose(c.cpu(), torch.tensor([[2., 1.]]), atol=1e-6)
    w = torch.tensor([[1., -1., 0., 1.], [0., 1., 1., -1.], [1., 0., -1., 0.]], device=DEV)
    x = torch.tensor([[0.5, -0.25, 2.0, 1.0]], device=DEV)
    c = torch.empty(1, 3, device=DEV)
    lib.gemm_generic(x, w, c)
    assert torch.allclose(c.cpu(), torch.tensor([[1.75, 0.75, -1.5]]), atol=1e-5)
    # the same through the matrix cores (K padded to 8 with zeros; values exact in bfloat16)
    wb = torch.zeros(3, 8, device=DEV, dtype=torch.bfloat16)
    wb[:, :4] = w.bfloat16()
    xb = torch.zeros(1, 8, device=DEV, dtype=torch.bfloat16)
    xb[:, :4] = x.bfloat16()
    lib.gemm_bf16(xb, wb, c, 0)
    assert torch.allclose(c.cpu(), torch.tensor([[1.75, 0.75, -1.5]]), atol=1e-5)


@pytest.mark.parametrize("m,n,k", [(1, 7, 5), (3, 130, 67), (65, 64, 16), (130, 200, 333), (1, 130, 64), (8, 1000, 2052),
                                   (16, 33, 4096), (5, 300, 1028), (4, 17, 4), (17, 50, 64), (17, 50, 60), (300, 200, 336),
                                   (129, 1000, 16), (2048, 130, 256)])
def test_gemm_generic_f32(lib, m, n, k):
    g = torch.Generator().manual_seed(m * 1000 + n)
    a = torch.randn(m, k, generator=g)
    w = torch.randn(n, k, generator=g)
    c = torch.empty(m, n, device=DEV)
    lib.gemm_generic(a.to(DEV), w.to(DEV), c)
    assert _rel(c, a.double() @ w.double().T) < 1e-5


@pytest.mark.parametrize("m", [1, 2, 8, 15, 16, 17, 33, 48, 64, 65, 127, 128, 200, 300])
@pytest.mark.parametrize("n,k", [(48, 64), (100, 136), (520, 1000), (4128, 512), (20000, 72), (40000, 264)])
def test_gemm_bf16(lib, m, n, k):
    if m > 128 and n >= 20000:
        pytest.skip("covered by smaller M")
    g = torch.Generator().manual_seed(m * 7 + n)
    a = torch.randn(m, k, generator=g).bfloat16()
    w = torch.randn(n, k, generator=g).bfloat16()
    want = a.double() @ w.double().T
    for out_dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 1e-2)):
        c = torch.full((m, n), float("nan"), device=DEV, dtype=out_dtype)
        lib.gemm_bf16(a.to(DEV), w.to(DEV), c, 0)
        assert _rel(c, want) < tol, (m, n, k, out_dtype)


@pytest.mark.parametrize("m", [1, 8, 20, 64, 100, 260])
@pytest.mark.parametrize("ff,k", [(16, 64), (336, 192), (8208, 136), (17000 // 16 * 16, 72)])
def test_gemm_bf16_gated(lib, m, ff, k):
    from helpers import interleave_gate_up
    g = torch.Generator().manual_seed(m + ff)
    x = torch.randn(m, k, generator=g).bfloat16()
    wg = (torch.randn(ff, k, generator=g) * 0.3).bfloat16()
    wu = (torch.randn(ff, k, generator=g) * 0.3).bfloat16()
    gate = x.double() @ wg.double().T
    want = gate / (1 + torch.exp(-gate)) * (x.double() @ wu.double().T)
    packed = interleave_gate_up(wg, wu).to(DEV)
    out = torch.full((m, ff), float("nan"), device=DEV, dtype=torch.bfloat16)
    lib.gemm_bf16(x.to(DEV), packed, out, 1)
    assert _rel(out, want) < 1e-2


@pytest.mark.parametrize("m,n,k,gated", [(513, 300, 128, False), (700, 14000, 192, False), (700, 14000, 64, False),
                                         (257, 41000, 320, False), (600, 14016, 128, True), (130, 96, 64, True),
                                         (1024, 16384, 128, False), (1000, 16384, 64, True),
                                         (100, 520, 1024, False), (130, 300, 4096, False), (600, 1000, 8192, False),
                                         (300, 4096, 2048, False), (129, 672, 256, True),
                                         (1500, 4000, 256, False), (250, 57344, 64, True), (2048, 4096, 192, False),
                                         (1030, 14300, 64, False), (1024, 28672 * 2, 64, True),
                                         (300, 4000, 8192, False), (520, 4100, 4096, False),
                                         (1100, 4000, 8192, False), (1300, 4096, 8192, False),
                                         (1300, 6100, 256, False)])
def test_gemm_bf16_tiles_loaded_straight_into_lds(lib, m, n, k, gated):
    """K a multiple of 64 and more than 64 tokens: the kernels whose tiles go from memory into
    LDS without passing registers, with all three tile sizes (128 x 128; 256 x 256 when its
    tiles fill whole rounds of workgroups, as with 4 x 64 of them; else 192 x 256), partial
    tiles at both edges, as few K tiles as one (fewer than the stages of the pipeline), and
    the products of 65..768 tokens whose tiles are too few, so that K is cut into slices
    (64-token tiles in 2 slices at 130 x 300 x 4096, 128 x 128 tiles in 2 at 600 x 1000 x 8192).
    Three cases make 192..256 tiles of 256 rows x 128 tokens, which then run in one round, with
    partial tiles at both edges and the gated epilogue; the last two make fewer rounds of 320-row
    tiles than of 256-row ones (5 x 45 = 225 against 5 x 56 = 280, and 4 x 180 against 4 x 224).
    The last five are tiles too few for a round whose K is cut: 48 tiles of 256 x 128 in 4 slices,
    85 in 2, 105 tiles of 192 x 256 in 2, 96 of 256 x 256 in 2, and 192 tiles of 192 x 256 uncut."""
    from helpers import interleave_gate_up
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    if gated:
        ff = n // 2
        wg = (torch.randn(ff, k, generator=g) * 0.3).bfloat16()
        wu = (torch.randn(ff, k, generator=g) * 0.3).bfloat16()
        gate = x.double() @ wg.double().T
        want = gate / (1 + torch.exp(-gate)) * (x.double() @ wu.double().T)
        out = torch.full((m, ff), float("nan"), device=DEV, dtype=torch.bfloat16)
        lib.gemm_bf16(x.to(DEV), interleave_gate_up(wg, wu).to(DEV), out, 1)
        assert _rel(out, want) < 1e-2
    else:
        w = torch.randn(n, k, generator=g).bfloat16()
        want = x.double() @ w.double().T
        out = torch.full((m, n), float("nan"), device=DEV, dtype=torch.float32)
        lib.gemm_bf16(x.to(DEV), w.to(DEV), out, 0)
        assert _rel(out, want) < 2e-5
        out16 = torch.full((m, n), float("nan"), device=DEV, dtype=torch.bfloat16)
        lib.gemm_bf16(x.to(DEV), w.to(DEV), out16, 0)
        assert _rel(out16, want) < 1e-2


# ------------------------------------------------------------------------ elementwise
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_gather(lib, dtype):
    table = torch.randn(37, 50).to(dtype)
    ids = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32)
    out = torch.empty(5, 50, device=DEV)
    lib.embed_gather(table.to(DEV), ids.to(DEV), out)
    assert torch.equal(out.cpu(), table.float()[ids.long()])


@pytest.mark.parametrize("width,eps", [(50, 1e-5), (1000, 1e-6), (4100, 1e-2), (4096, 1e-5), (12000, 1e-5)])
def test_add_rmsnorm(lib, width, eps):
    g = torch.Generator().manual_seed(width)
    x = torch.randn(6, width, generator=g) * 1e-2        # small, so that eps matters
    d = torch.randn(6, width, generator=g) * 1e-2
    w = 1 + 0.1 * torch.randn(width, generator=g)

    def ref(v):
        v = v.double()
        return v * w.double() / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)

    xd = x.to(DEV).clone()
    out = torch.empty(6, width, device=DEV)
    lib.add_rmsnorm(xd, None, w.to(DEV), eps, None, out)
    assert _rel(out, ref(x)) < 1e-6
    assert torch.equal(xd.cpu(), x)
    lib.add_rmsnorm(xd, d.to(DEV), w.to(DEV), eps, None, out)          # adds in place
    assert _rel(out, ref(x + d)) < 1e-6
    assert torch.allclose(xd.cpu(), x + d, atol=0, rtol=0)
    rows = torch.tensor([4, 1, 1], dtype=torch.int32, device=DEV)       # gather: x stays
    xd2 = x.to(DEV).clone()
    outb = torch.empty(3, width, device=DEV, dtype=torch.bfloat16)
    lib.add_rmsnorm(xd2, d.to(DEV), w.to(DEV), eps, rows, outb)
    assert torch.equal(xd2.cpu(), x)
    assert _rel(outb, ref(x + d)[[4, 1, 1]]) < 5e-3
    # a wrong eps, or eps outside the root, must show at this scale
    wrong = (x + d).double() * w.double() / (torch.sqrt(((x + d).double() ** 2).mean(-1, keepdim=True)) + eps)
    assert _rel(out, wrong) > 1e-4


def test_swiglu(lib):
    g = torch.Generator().manual_seed(3)
    gu = torch.randn(5, 2 * 77, generator=g) * 4
    out = torch.empty(5, 77, device=DEV)
    lib.swiglu(gu.to(DEV), out)
    gate, up = gu[:, :77].double(), gu[:, 77:].double()
    assert _rel(out, gate / (1 + torch.exp(-gate)) * up) < 1e-6


# ------------------------------------------------------------------------ rope + cache write, attention
def _paged_setup(lens_past, q_lens, n_kv, d, dtype, n_pages=64, seed=0):
    """Random q/k/v for a ragged batch and a shuffled page assignment."""
    g = torch.Generator().manual_seed(seed)
    b = len(q_lens)
    total = [p + q for p, q in zip(lens_past, q_lens)]
    perm = torch.randperm(n_pages, generator=g).tolist()
    tables, used = [], 0
    for t in total:
        n = (t + 63) // 64
        tables.append(perm[used:used + n])
        used += n
    width = max(len(t) for t in tables)
    bt = torch.tensor([t + [0] * (width - len(t)) for t in tables], dtype=torch.int32)
    tok_seq = torch.tensor([i for i, q in enumerate(q_lens) for _ in range(q)], dtype=torch.int32)
    tok_pos = torch.tensor([p + j for p, q in zip(lens_past, q_lens) for j in range(q)], dtype=torch.int32)
    return g, bt, tok_seq, tok_pos, total


def _fill_pages(k_full, v_full, bt, n_pages, n_kv, d, dtype):
    """k_full[b]: [len, n_kv, d] -> page tensors filled with NaN where nothing is stored."""
    kp = torch.full((n_pages, n_kv, 64, d), float("nan"), dtype=dtype)
    vp = torch.full((n_pages, n_kv, 64, d), float("nan"), dtype=dtype)
    for b, (kf, vf) in enumerate(zip(k_full, v_full)):
        for p in range(kf.shape[0]):
            page = int(bt[b, p // 64])
            kp[page, :, p % 64] = kf[p].to(dtype)
            vp[page, :, p % 64] = vf[p].to(dtype)
    return kp, vp


def _is_rounding_of(stored, exact, size):
    """Whether each bfloat16 in `stored` is the rounding of a number within 1e-6 * size of the
    float64 in `exact`: what 32-bit arithmetic on operands of that size may leave before the one
    rounding, and no more."""
    exact = exact.double()
    err = (stored.double() - exact).abs()
    ulp = torch.exp2(torch.floor(torch.log2(exact.abs().clamp_min(1e-30))) - 7)
    return bool((err <= 0.5 * ulp + 1e-6 * size).all())


def _attention_ref(q, k_full, v_full, tok_seq, tok_pos, n_heads, n_kv, scale, window):
    out = torch.zeros(q.shape[0], n_heads * q.shape[2], dtype=torch.float64)
    d = q.shape[2]
    for t in range(q.shape[0]):
        b, pos = int(tok_seq[t]), int(tok_pos[t])
        lo = 0 if not window else max(0, pos - window + 1)
        for h in range(n_heads):
            kvh = h // (n_heads // n_kv)
            s = (k_full[b][lo:pos + 1, kvh].double() @ q[t, h].double()) * scale
            p = torch.softmax(s, 0)
            out[t, h * d:(h + 1) * d] = p @ v_full[b][lo:pos + 1, kvh].double()
    return out


@pytest.mark.parametrize("style", [0, 1])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d", [48, 20])
def test_rope_kv_write(lib, style, dtype, d):
    """Head size 48: the kernel that takes four pairs a thread; 20 (no multiple of 8): one pair a thread."""
    n_heads, n_kv = 3, 3
    past, q_lens = [0, 70, 5], [3, 2, 60]
    g, bt, tok_seq, tok_pos, total = _paged_setup(past, q_lens, n_kv, d, dtype)
    t = sum(q_lens)
    qkv = torch.randn(t, (n_heads + 2 * n_kv) * d, generator=g)
    inv = 1.0 / (10000.0 ** (torch.arange(d // 2).double() * 2 / d))
    ang = torch.arange(200).double()[:, None] * inv[None]
    cos, sin = torch.cos(ang).float(), torch.sin(ang).float()
    kp = torch.zeros(64, n_kv, 64, d, dtype=dtype, device=DEV)
    vp = torch.zeros_like(kp)
    qo = torch.empty(t, n_heads, d, dtype=dtype, device=DEV)
    lib.rope_kv_write(qkv.to(DEV), cos.to(DEV), sin.to(DEV), style, qo, kp, vp, tok_pos.to(DEV), tok_seq.to(DEV),
                      bt.to(DEV), n_heads, n_kv, d)
    tol = 1e-6 if dtype == torch.float32 else 5e-3
    for i in range(t):
        pos, b = int(tok_pos[i]), int(tok_seq[i])
        heads = qkv[i].double().view(n_heads + 2 * n_kv, d)
        z = torch.polar(torch.ones(d // 2, dtype=torch.float64), ang[pos])          # exp(i * pos * inv)
        if style == 0:
            rot = torch.view_as_real(torch.view_as_complex(heads[:n_heads + n_kv].reshape(-1, d // 2, 2)) * z)
            rot = rot.reshape(-1, d)
        else:
            c = torch.complex(heads[:n_heads + n_kv, :d // 2], heads[:n_heads + n_kv, d // 2:]) * z
            rot = torch.cat([c.real, c.imag], dim=1)
        assert _rel(qo[i], rot[:n_heads]) < tol
        page = int(bt[b, pos // 64])
        assert _rel(kp[page, :, pos % 64], rot[n_heads:]) < tol
        assert _rel(vp[page, :, pos % 64], heads[n_heads + n_kv:]) < tol
    # qkv as the terms of a product whose K was cut into slices: added up in their order
    for n_terms in (2, 7):
        terms = torch.randn(n_terms, *qkv.shape, generator=g)
        total = terms[0].clone()
        for p in range(1, n_terms):
            total += terms[p]
        kp1, vp1, qo1 = torch.zeros_like(kp), torch.zeros_like(vp), torch.empty_like(qo)
        kp2, vp2, qo2 = torch.zeros_like(kp), torch.zeros_like(vp), torch.empty_like(qo)
        lib.rope_kv_write(total.to(DEV), cos.to(DEV), sin.to(DEV), style, qo1, kp1, vp1, tok_pos.to(DEV),
                          tok_seq.to(DEV), bt.to(DEV), n_heads, n_kv, d)
        lib.rope_kv_write(terms.to(DEV), cos.to(DEV), sin.to(DEV), style, qo2, kp2, vp2, tok_pos.to(DEV),
                          tok_seq.to(DEV), bt.to(DEV), n_heads, n_kv, d)
        assert torch.equal(qo1, qo2) and torch.equal(kp1, kp2) and torch.equal(vp1, vp2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_heads,n_kv,d,window", [(3, 3, 16, 0), (6, 2, 48, 0), (4, 1, 80, 37), (5, 5, 256, 0)])
def test_attention_generic(lib, dtype, n_heads, n_kv, d, window):
    past, q_lens = [0, 70, 129, 63], [5, 1, 3, 66]
    g, bt, tok_seq, tok_pos, total = _paged_setup(past, q_lens, n_kv, d, dtype, seed=d)
    k_full = [torch.randn(n, n_kv, d, generator=g).to(dtype) for n in total]
    v_full = [torch.randn(n, n_kv, d, generator=g).to(dtype) for n in total]
    q = torch.randn(sum(q_lens), n_heads, d, generator=g).to(dtype)
    kp, vp = _fill_pages(k_full, v_full, bt, 64, n_kv, d, dtype)
    out = torch.empty(q.shape[0], n_heads * d, dtype=dtype, device=DEV)
    scale = 1 / math.sqrt(d)
    lib.attention_generic(q.to(DEV), kp.to(DEV), vp.to(DEV), out, tok_pos.to(DEV), tok_seq.to(DEV), bt.to(DEV),
                          n_heads, n_kv, d, scale, window)
    want = _attention_ref(q, k_full, v_full, tok_seq, tok_pos, n_heads, n_kv, scale, window)
    assert _rel(out, want) < (2e-6 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("n_heads,n_kv,d,window", [(4, 1, 128, 0), (8, 8, 64, 0), (6, 3, 128, 0), (8, 1, 64, 100),
                                                  (2, 2, 128, 70)])
def test_attention_prefill_bf16(lib, n_heads, n_kv, d, window):
    past, q_lens = [0, 70, 129, 0, 200], [150, 33, 3, 64, 1]
    dtype = torch.bfloat16
    g, bt, tok_seq, tok_pos, total = _paged_setup(past, q_lens, n_kv, d, dtype, seed=n_heads)
    k_full = [torch.randn(n, n_kv, d, generator=g).to(dtype) for n in total]
    v_full = [torch.randn(n, n_kv, d, generator=g).to(dtype) for n in total]
    q = (torch.randn(sum(q_lens), n_heads, d, generator=g) * 2).to(dtype)
    kp, vp = _fill_pages(k_full, v_full, bt, 64, n_kv, d, dtype)
    out = torch.full((q.shape[0], n_heads * d), float("nan"), dtype=dtype, device=DEV)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    scale = 1 / math.sqrt(d)
    lib.attention_prefill_bf16(q.to(DEV), kp.to(DEV), vp.to(DEV), out, cu.to(DEV),
                               torch.tensor(past, dtype=torch.int32, device=DEV), bt.to(DEV), len(q_lens),
                               max(q_lens), n_heads, n_kv, d, scale, window)
    want = _attention_ref(q, k_full, v_full, tok_seq, tok_pos, n_heads, n_kv, scale, window)
    assert _rel(out, want) < 1.5e-2


@pytest.mark.parametrize("waves", [0, 4, 8])
@pytest.mark.parametrize("n_heads,n_kv,d,t,window", [(24, 24, 64, 1536, 0), (32, 8, 128, 1100, 0), (8, 2, 128, 2500, 300),
                                                    (4, 4, 64, 700, 0), (6, 3, 128, 333, 70)])
def test_attention_prefill_of_a_long_prompt(lib, waves, n_heads, n_kv, d, t, window):
    """One prompt of a thousand tokens and more, where the order in which the workgroups take
    the blocks of queries matters: between 257 and 512 workgroups a sequence (288, 280 and 316
    in the first three cases) the heaviest and the lightest blocks are paired; the last case
    has fewer.  waves = 8: the kernel with twice the queries per workgroup, which the
    library takes only beyond 8,192 tokens.  Every row of the output is compared."""
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(t + n_heads)
    n_pages = (t + 63) // 64
    q = (torch.randn(t, n_heads, d, generator=g) * 1.5).to(dtype)
    k = torch.randn(t, n_kv, d, generator=g).to(dtype)
    v = torch.randn(t, n_kv, d, generator=g).to(dtype)
    order = torch.randperm(n_pages, generator=g).to(torch.int32)          # the pages lie anywhere
    kp = torch.full((n_pages, n_kv, 64, d), float("nan"), dtype=dtype)
    vp = torch.full((n_pages, n_kv, 64, d), float("nan"), dtype=dtype)
    for pg in range(n_pages):
        rows = slice(64 * pg, min(64 * pg + 64, t))
        kp[int(order[pg]), :, :rows.stop - rows.start] = k[rows].transpose(0, 1)
        vp[int(order[pg]), :, :rows.stop - rows.start] = v[rows].transpose(0, 1)
    out = torch.full((t, n_heads * d), float("nan"), dtype=dtype, device=DEV)
    cu = torch.tensor([0, t], dtype=torch.int32, device=DEV)
    scale = 1 / math.sqrt(d)
    lib._lib.rb_tune_prefill_waves(waves)
    try:
        lib.attention_prefill_bf16(q.to(DEV), kp.to(DEV), vp.to(DEV), out, cu,
                                   torch.zeros(1, dtype=torch.int32, device=DEV), order.view(1, -1).to(DEV), 1, t,
                                   n_heads, n_kv, d, scale, window)
    finally:
        lib._lib.rb_tune_prefill_waves(0)
    # plain attention in float64 (on the GPU, for its speed)
    qd, kd, vd = q.to(DEV).double(), k.to(DEV).double(), v.to(DEV).double()
    pos = torch.arange(t, device=DEV)
    seen = pos[None, :] <= pos[:, None]
    if window:
        seen &= pos[None, :] > pos[:, None] - window
    want = torch.empty(t, n_heads, d, dtype=torch.float64, device=DEV)
    for h in range(n_heads):
        kvh = h // (n_heads // n_kv)
        scores = (qd[:, h] @ kd[:, kvh].T) * scale
        scores = scores.masked_fill(~seen, float("-inf"))
        want[:, h] = torch.softmax(scores, dim=1) @ vd[:, kvh]
    got = out.double().view(t, n_heads, d)
    assert bool(torch.isfinite(got).all())
    err = (got - want).abs().amax(dim=(1, 2)) / want.abs().amax()
    assert float(err.max()) < 1.5e-2, int(err.argmax())


@pytest.fixture
def decode_kernel(lib, request):
    """"auto": the kernel the library picks for the group size; "matrix": the matrix-core
    decode kernel whatever the group size."""
    lib._lib.rb_tune_decode_mfma(1 if request.param == "matrix" else 0)
    yield request.param
    lib._lib.rb_tune_decode_mfma(0)


_DECODE_CASES = [(4, 1, 128, 0, 3), (8, 8, 64, 0, 1), (8, 4, 128, 0, 8), (8, 1, 64, 90, 2), (2, 2, 128, 65, 5),
                 (6, 2, 128, 0, 3), (16, 1, 64, 0, 2), (10, 2, 128, 70, 2), (7, 1, 64, 0, 4), (12, 1, 128, 130, 1),
                 (8, 8, 128, 0, 16)]          # the last one: 768 workgroups, where keys are read past the caches


@pytest.mark.parametrize("decode_kernel", ["auto", "matrix"], indirect=True)
@pytest.mark.parametrize("n_heads,n_kv,d,window,n_splits", _DECODE_CASES)
def test_attention_decode_bf16(lib, n_heads, n_kv, d, window, n_splits, decode_kernel):
    past, q_lens = [0, 70, 129, 63, 64, 300], [1, 1, 1, 1, 1, 1]
    dtype = torch.bfloat16
    g, bt, tok_seq, tok_pos, total = _paged_setup(past, q_lens, n_kv, d, dtype, seed=n_heads + 1)
    k_full = [torch.randn(n, n_kv, d, generator=g).to(dtype) for n in total]
    v_full = [torch.randn(n, n_kv, d, generator=g).to(dtype) for n in total]
    q = (torch.randn(len(q_lens), n_heads, d, generator=g) * 2).to(dtype)
    kp, vp = _fill_pages(k_full, v_full, bt, 64, n_kv, d, dtype)
    out = torch.full((q.shape[0], n_heads * d), float("nan"), dtype=dtype, device=DEV)
    ws = torch.full((len(q_lens) * n_heads * n_splits * (d + 2),), float("nan"), device=DEV)
    scale = 1 / math.sqrt(d)
    lib.attention_decode_bf16(q.to(DEV), kp.to(DEV), vp.to(DEV), out, tok_pos.to(DEV), bt.to(DEV), n_heads, n_kv, d,
                              scale, window, n_splits, ws)
    want = _attention_ref(q, k_full, v_full, tok_seq, tok_pos, n_heads, n_kv, scale, window)
    assert _rel(out, want) < 1e-2


def test_far_key_stands_out(lib):
    """One key among hundreds, scaled so that its score dominates: the output must be that
    key's value, wherever it lies (first page, page edge, last position)."""
    n_heads, n_kv, d = 4, 1, 128
    dtype = torch.bfloat16
    total = 700
    for target in (0, 63, 64, 511, 698, 699):
        g, bt, tok_seq, tok_pos, _ = _paged_setup([total - 1], [1], n_kv, d, dtype, seed=target)
        k = torch.randn(total, n_kv, d, generator=g) * 0.1
        v = torch.randn(total, n_kv, d, generator=g)
        q = torch.randn(1, n_heads, d, generator=g) * 0.1
        k[target, 0] = 40 * q[0, 1] / q[0, 1].norm()          # head 1 looks at `target`
        q[0, 1] = 40 * q[0, 1] / q[0, 1].norm()
        kp, vp = _fill_pages([k], [v], bt, 64, n_kv, d, dtype)
        scale = 1 / math.sqrt(d)
        outs = []
        out = torch.empty(1, n_heads * d, dtype=dtype, device=DEV)
        lib.attention_generic(q.to(dtype).to(DEV), kp.to(DEV), vp.to(DEV), out, tok_pos.to(DEV), tok_seq.to(DEV),
                              bt.to(DEV), n_heads, n_kv, d, scale, 0)
        outs.append(out.clone())
        ws = torch.empty(n_heads * 4 * (d + 2), device=DEV)
        for mode in (0, 1):             # the vector kernel, the matrix-core kernel
            lib._lib.rb_tune_decode_mfma(mode)
            try:
                lib.attention_decode_bf16(q.to(dtype).to(DEV), kp.to(DEV), vp.to(DEV), out, tok_pos.to(DEV),
                                          bt.to(DEV), n_heads, n_kv, d, scale, 0, 4, ws)
            finally:
                lib._lib.rb_tune_decode_mfma(0)
            outs.append(out.clone())
        cu = torch.tensor([0, 1], dtype=torch.int32, device=DEV)
        lib.attention_prefill_bf16(q.to(dtype).to(DEV), kp.to(DEV), vp.to(DEV), out, cu,
                                   torch.tensor([total - 1], dtype=torch.int32, device=DEV), bt.to(DEV), 1, 1,
                                   n_heads, n_kv, d, scale, 0)
        outs.append(out.clone())
        for o in outs:
            got = o[0, d:2 * d].float().cpu()
            assert (got - v[target, 0].to(dtype).float()).abs().max() < 2e-2, target


# ------------------------------------------------------------------------ sampling
def test_sample_greedy_and_inverse_cdf(lib):
    from plain_llama import sample_token
    g = torch.Generator().manual_seed(11)
    logits = torch.randn(7, 9001, generator=g) * 3        # three chunks, the last one short
    logits[2, 5] = logits[2, 8900] = 50.0                # equal maxima: the lowest index wins
    logits[3, 17] = float("nan")
    tokens = torch.empty(7, dtype=torch.int32, device=DEV)
    lib.sample(logits.to(DEV), None, None, tokens)
    want = [int(torch.nan_to_num(r, nan=-float("inf")).argmax()) for r in logits]
    want[2] = 5
    assert tokens.tolist() == want
    temps = torch.tensor([0.8, 0.0, 1.5, 0.3, 1.0, 0.8, 2.0])
    us = torch.tensor([0.0, 0.5, 0.999999, 0.25, 0.5, 0.73, 0.1])
    logits[4, 4096:8192] += 6.0                          # most of the mass in the middle chunk
    lib.sample(logits.to(DEV), temps.to(DEV), us.to(DEV), tokens)
    for r in range(7):
        row = torch.nan_to_num(logits[r], nan=-float("inf"))
        assert tokens[r].item() == sample_token(row, float(temps[r]), float(us[r])), r


@pytest.mark.parametrize("decode_kernel", ["auto", "matrix"], indirect=True)
@pytest.mark.parametrize("style", [0, 1])
@pytest.mark.parametrize("n_heads,n_kv,d,window,n_splits", _DECODE_CASES + [(4, 2, 64, 0, 32)])
def test_attention_decode_fused_bf16(lib, n_heads, n_kv, d, window, n_splits, style, decode_kernel):
    """Rotation, cache write and attention in one kernel (and the combination of splits),
    against the separate steps computed plainly; called three times in a row."""
    past, q_lens = [0, 70, 129, 63, 64, 300], [1, 1, 1, 1, 1, 1]
    dtype = torch.bfloat16
    nb = len(past)
    g, bt, tok_seq, tok_pos, total = _paged_setup(past, q_lens, n_kv, d, dtype, seed=n_heads + 5)
    k_past = [torch.randn(n, n_kv, d, generator=g).to(dtype) for n in past]
    v_past = [torch.randn(n, n_kv, d, generator=g).to(dtype) for n in past]
    inv = 1.0 / (10000.0 ** (torch.arange(d // 2).double() * 2 / d))
    ang = torch.arange(400).double()[:, None] * inv[None]
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    scale = 1 / math.sqrt(d)
    ws = torch.full((nb * n_heads * n_splits * (d + 2),), float("nan"), device=DEV)
    for call in range(3):
        qkv = torch.randn(nb, (n_heads + 2 * n_kv) * d, generator=g) * 1.5
        # plain: rotate q and k, round to bfloat16, append k and v, attend
        rot = torch.empty(nb, n_heads + n_kv, d, dtype=torch.float64)
        for b in range(nb):
            heads = qkv[b].double().view(n_heads + 2 * n_kv, d)[:n_heads + n_kv]
            z = torch.polar(torch.ones(d // 2, dtype=torch.float64), ang[past[b]])
            if style == 0:
                rot[b] = torch.view_as_real(torch.view_as_complex(heads.reshape(-1, d // 2, 2)) * z).reshape(-1, d)
            else:
                c = torch.complex(heads[:, :d // 2], heads[:, d // 2:]) * z
                rot[b] = torch.cat([c.real, c.imag], dim=1)
        q = rot[:, :n_heads].to(dtype)
        k_new = rot[:, n_heads:].to(dtype)
        v_new = qkv.view(nb, n_heads + 2 * n_kv, d)[:, n_heads + n_kv:].to(dtype)
        k_full = [torch.cat([k_past[b], k_new[b:b + 1]]) for b in range(nb)]
        v_full = [torch.cat([v_past[b], v_new[b:b + 1]]) for b in range(nb)]
        want = _attention_ref(q, k_full, v_full, tok_seq, tok_pos, n_heads, n_kv, scale, window)
        kp, vp = _fill_pages(k_past, v_past, bt, 64, n_kv, d, dtype)       # the new position holds NaN
        kp, vp = kp.to(DEV), vp.to(DEV)
        out = torch.full((nb, n_heads * d), float("nan"), dtype=dtype, device=DEV)
        lib.attention_decode_fused_bf16(qkv.to(DEV), cos, sin, style, kp, vp, out, tok_pos.to(DEV), bt.to(DEV),
                                        n_heads, n_kv, d, scale, window, n_splits, ws)
        assert _rel(out, want) < 1e-2, call
        for b in range(nb):
            page, off = int(bt[b, past[b] // 64]), past[b] % 64
            assert _is_rounding_of(kp[page, :, off].cpu(), rot[b, n_heads:], float(qkv[b].abs().max()))
            assert torch.equal(vp[page, :, off].cpu(), v_new[b])
        if call == 0:
            # qkv as 6 terms that add up (in their order) to the same numbers: the same result, bit for bit
            parts = torch.randn(5, *qkv.shape, generator=g)
            rest = qkv.clone()
            for p in range(5):
                rest -= parts[p]
            terms = torch.cat([parts, rest[None]])
            total = terms[0].clone()
            for p in range(1, 6):
                total += terms[p]
            kp1, vp1 = _fill_pages(k_past, v_past, bt, 64, n_kv, d, dtype)
            kp2, vp2 = _fill_pages(k_past, v_past, bt, 64, n_kv, d, dtype)
            kp1, vp1, kp2, vp2 = kp1.to(DEV), vp1.to(DEV), kp2.to(DEV), vp2.to(DEV)
            out1, out2 = torch.empty_like(out), torch.empty_like(out)
            lib.attention_decode_fused_bf16(total.to(DEV), cos, sin, style, kp1, vp1, out1, tok_pos.to(DEV),
                                            bt.to(DEV), n_heads, n_kv, d, scale, window, n_splits, ws)
            lib.attention_decode_fused_bf16(terms.to(DEV), cos, sin, style, kp2, vp2, out2, tok_pos.to(DEV),
                                            bt.to(DEV), n_heads, n_kv, d, scale, window, n_splits, ws)
            assert torch.equal(out1, out2)
            for b in range(nb):
                page, off = int(bt[b, past[b] // 64]), past[b] % 64
                assert torch.equal(kp1[page, :, off], kp2[page, :, off])
                assert torch.equal(vp1[page, :, off], vp2[page, :, off])


@pytest.mark.parametrize("m", [17, 31, 48, 64])
@pytest.mark.parametrize("n,k,epi", [(4096, 1024, 0), (520, 512, 0), (200, 128, 0), (100, 64, 0), (333, 192, 0),
                                     (6144, 4096, 0), (672, 256, 1), (8208 * 2, 384, 1)])
def test_gemm_bf16_17_to_64_tokens(lib, m, n, k, epi):
    """17..64 tokens with K a multiple of 64: one token tile, W streamed through LDS, with
    and without K cut into slices over workgroups whose slabs are added up afterwards."""
    g = torch.Generator().manual_seed(m * 3 + n)
    a = torch.randn(m, k, generator=g).bfloat16()
    if epi:
        from helpers import interleave_gate_up
        ff = n // 2
        wg = (torch.randn(ff, k, generator=g) * 0.3).bfloat16()
        wu = (torch.randn(ff, k, generator=g) * 0.3).bfloat16()
        gate = a.double() @ wg.double().T
        want = gate / (1 + torch.exp(-gate)) * (a.double() @ wu.double().T)
        w = interleave_gate_up(wg, wu)
        out = torch.full((m, ff), float("nan"), device=DEV, dtype=torch.bfloat16)
        tol = 1e-2
    else:
        w = torch.randn(n, k, generator=g).bfloat16()
        want = a.double() @ w.double().T
        out = torch.full((m, n), float("nan"), device=DEV, dtype=torch.float32)
        tol = 2e-5
    lib.gemm_bf16(a.to(DEV), w.to(DEV), out, epi)
    assert _rel(out, want) < tol
    if not epi:
        out16 = torch.full((m, n), float("nan"), device=DEV, dtype=torch.bfloat16)
        lib.gemm_bf16(a.to(DEV), w.to(DEV), out16, epi)
        assert _rel(out16, want) < 1e-2


def _prepared(x, gain):
    """What epilogue 3 leaves for the norm after it: bf16(x * gain) and the sums of x^2 over
    every 16 columns, computed the plain way."""
    t, e = x.shape
    padded = torch.zeros(t, (e + 15) // 16 * 16, dtype=torch.float64)
    padded[:, :e] = x.double() ** 2
    return (x * gain).bfloat16(), padded.view(t, -1, 16).sum(dim=2).float()


@pytest.mark.parametrize("m,n,k", [(1, 48, 64), (8, 4096, 4096), (16, 100, 136), (5, 6144, 1024), (8, 8208, 512),
                                   (3, 9000, 4096), (7, 16400, 8192), (16, 20000, 200), (2, 12288, 1536),
                                   (4, 520, 14336), (9, 264, 8200)])
def test_gemm_bf16_few_tokens_folds_sum_and_norm(lib, m, n, k):
    """The decode products with their neighbours folded in.  As tokens: rows that a product left
    for a norm (bf16(x * gain) and the sums of x^2 in parts of 16 columns), all of them or chosen
    ones; the result is that of the normalised rows.  As epilogues: the product added to a
    float32 matrix, and that with the rows for the next norm left behind.  Sizes cover the
    streaming kernel with and without bounds checks (K a multiple of 128 or not), 1, 2 and 4 row
    tiles per wave, a last tile of fewer than 16 columns, counts of sums that are no multiple of
    4 (K = 136, 200, 8200), more sums than the wide loads take (K = 14336), and the kernel that
    keeps the tokens in registers (more than 8192 rows of W, K a multiple of 512 up to 4096).
    The matrix cores see bf16(x * gain), which the first reference repeats; the second is the
    norm as its own kernel computes it, rounded after the root."""
    from helpers import interleave_gate_up
    assert lib.gemm_bf16_few_ok(m, n, k)
    g = torch.Generator().manual_seed(m * 11 + n + k)
    eps = 1e-3
    pool = torch.randn(m + 5, k, generator=g) * 0.05          # small, so that eps matters
    gain = 1 + 0.2 * torch.randn(k, generator=g)
    w = (torch.randn(n, k, generator=g) * 0.5).bfloat16()
    gained, squares = _prepared(pool, gain)
    for rows in (None, torch.randperm(m + 5, generator=g)[:m].to(torch.int32)):
        sel = slice(0, m) if rows is None else rows.long()
        a = gained[:m].contiguous() if rows is None else gained
        sq = squares[:m].contiguous() if rows is None else squares
        picked = pool[sel]
        scale = 1.0 / torch.sqrt((picked.double() ** 2).mean(dim=1, keepdim=True) + eps)
        want = (gained[sel].double() @ w.double().T) * scale
        loose = (picked.double() * gain.double() * scale).float().bfloat16().double() @ w.double().T
        out = torch.full((m, n), float("nan"), device=DEV, dtype=torch.float32)
        lib.gemm_bf16_few(a.to(DEV), w.to(DEV), out, 0, squares=sq.to(DEV), eps=eps,
                          rows=None if rows is None else rows.to(DEV))
        assert _rel(out, want) < 2e-5, (m, n, k, rows is None)
        assert _rel(out, loose) < 1e-2
    # bfloat16 tokens: plain, added to the output, and with the rows for the next norm
    a = torch.randn(m, k, generator=g).bfloat16()
    product = a.double() @ w.double().T
    plain = torch.full((m, n), float("nan"), device=DEV, dtype=torch.float32)
    lib.gemm_bf16_few(a.to(DEV), w.to(DEV), plain, 0)
    same = torch.full((m, n), float("nan"), device=DEV, dtype=torch.float32)
    lib.gemm_bf16(a.to(DEV), w.to(DEV), same, 0)
    assert torch.equal(plain, same)
    base = torch.randn(m, n, generator=g)
    acc = base.to(DEV)
    lib.gemm_bf16_few(a.to(DEV), w.to(DEV), acc, 2)
    assert _rel(acc, base.double() + product) < 2e-5
    next_gain = 1 + 0.2 * torch.randn(n, generator=g)
    acc3 = base.to(DEV)
    left = torch.full((m, n), float("nan"), device=DEV, dtype=torch.bfloat16)
    left_sq = torch.full((m, (n + 15) // 16), float("nan"), device=DEV)
    lib.gemm_bf16_few(a.to(DEV), w.to(DEV), acc3, 3, gain=next_gain.to(DEV), gained=left, squares_out=left_sq)
    assert torch.equal(acc3, acc)
    want_left, want_sq = _prepared(acc3.cpu(), next_gain)
    assert torch.equal(left.cpu(), want_left)
    assert _rel(left_sq, want_sq) < 1e-6
    # prepared rows into the gated epilogue
    if n % 32 == 0:
        ff = n // 2
        wg, wu = w[:ff], w[ff:]
        scale = 1.0 / torch.sqrt((pool[:m].double() ** 2).mean(dim=1, keepdim=True) + eps)
        gate = (gained[:m].double() @ wg.double().T) * scale
        want = gate / (1 + torch.exp(-gate)) * ((gained[:m].double() @ wu.double().T) * scale)
        out = torch.full((m, ff), float("nan"), device=DEV, dtype=torch.bfloat16)
        lib.gemm_bf16_few(gained[:m].contiguous().to(DEV), interleave_gate_up(wg, wu).to(DEV), out, 1,
                          squares=squares[:m].contiguous().to(DEV), eps=eps)
        assert _rel(out, want) < 1e-2


@pytest.mark.parametrize("m,n,k", [(40, 4096, 4096), (64, 512, 14336), (300, 1000, 8192), (20, 96, 64), (8, 64, 256)])
def test_gemm_terms_and_the_norm_that_adds_them(lib, m, n, k):
    """A product left as the partial sums of its K slices, and the norm that adds them to the
    stream: the same sums, bit for bit, as the product summed by its own kernel and then
    added (the terms are added up in the same order).  Sizes with several terms (few tiles, a
    long K) and with one."""
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).bfloat16().to(DEV)
    w = (torch.randn(n, k, generator=g) * 0.1).bfloat16().to(DEV)
    whole = torch.empty(m, n, device=DEV)
    lib.gemm_bf16(a, w, whole, 0)
    terms = lib.gemm_bf16_terms(a, w)
    assert terms.shape[0] == lib.gemm_bf16_terms_count(m, n, k) and terms.shape[1:] == (m, n)
    if (m, n, k) in ((40, 4096, 4096), (64, 512, 14336), (300, 1000, 8192)):
        assert terms.shape[0] > 1
    total = torch.zeros(m, n, device=DEV)
    for p in range(terms.shape[0]):
        total += terms[p]
    assert torch.equal(total, whole)
    gain = (1 + 0.1 * torch.randn(n, generator=g)).to(DEV)
    x0 = torch.randn(m, n, generator=g).to(DEV)
    for rows in (None, torch.tensor([m - 1, 0, 3], dtype=torch.int32, device=DEV)):
        r = m if rows is None else 3
        xa, xb = x0.clone(), x0.clone()
        ha = torch.empty(r, n, device=DEV, dtype=torch.bfloat16)
        hb = torch.empty(r, n, device=DEV, dtype=torch.bfloat16)
        lib.add_rmsnorm(xa, whole, gain, 1e-5, rows, ha)
        lib.add_rmsnorm(xb, terms, gain, 1e-5, rows, hb)
        # the stream bit for bit; the rows may differ by a rounding, since the squares of a row
        # are summed by more threads when there are terms to read
        assert torch.equal(xa, xb)
        assert float((ha.float() - hb.float()).abs().max()) <= 2 ** -7 * float(ha.float().abs().max())
        if rows is None:
            assert torch.equal(xa, x0 + whole)


@pytest.mark.parametrize("m,n,k,gated", [
    (512, 10240, 8192, False), (192, 8192, 28672, False), (1536, 4096, 14336, False), (384, 12288, 4096, False),
    (64, 4096, 11008, False),          # 172 K tiles: 8 slices do not divide them
    (48, 4096, 4096, False), (96, 57344, 8192, True), (256, 22016, 4096, True), (24, 22016, 4096, True),
    (700, 3072, 2048, False), (300, 5120, 13824, False),      # 216 K tiles: slices of 3 and 6
])
def test_products_of_the_model_shapes_with_the_planner_s_own_choice(lib, m, n, k, gated):
    """Products of the model shapes with whatever tile and number of K slices the planner picks,
    W stored fragment-major as the engine stores it, against a float32 product; deep products of
    few tokens must come in several slices (one slice would leave most of the GPU idle)."""
    min_terms = 2 if (not gated and m <= 512 and k >= 8192) else 1
    from helpers import fragment_major
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).bfloat16().to(DEV)
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16().to(DEV)
    wf = fragment_major(w)
    if gated:
        out = torch.full((m, n // 2), float("nan"), device=DEV, dtype=torch.bfloat16)
        lib.gemm_bf16(a, wf, out, 1, w_frag=True)
        wr = w.float().view(n // 32, 2, 16, k)
        gate = a.float() @ wr[:, 0].reshape(n // 2, k).T
        up = a.float() @ wr[:, 1].reshape(n // 2, k).T
        want = torch.nn.functional.silu(gate) * up
        assert _rel(out, want) < 1e-2
        return
    terms = lib.gemm_bf16_terms(a, wf, w_frag=True)
    assert terms.shape[0] >= min_terms and terms.shape[1:] == (m, n)
    want = a.float() @ w.float().T
    assert _rel(terms.sum(0), want) < 2e-3
    rows = lib.gemm_bf16_terms(a, w)                     # the same product with W as rows: the same bits
    assert torch.equal(rows, terms)


@pytest.mark.parametrize("units", [40, 96, 304])
def test_products_planned_for_another_number_of_compute_units(lib, units):
    """The planners told that the GPU has 40, 96 or 304 compute units (the count is their only input of the
    machine): other tiles, K slices, rows per wave and workgroup counts, the same products."""
    from helpers import fragment_major
    lib._lib.rb_tune_compute_units(units)
    try:
        for m, n, k, gated in ((1, 6144, 4096, False), (8, 28672, 4096, True), (16, 4096, 14336, False),
                               (40, 4096, 4096, False), (64, 512, 14336, False), (200, 12288, 1024, False),
                               (700, 22016, 2048, True), (1100, 4096, 8192, False)):
            g = torch.Generator().manual_seed(units + m + n + k)
            a = torch.randn(m, k, generator=g).bfloat16().to(DEV)
            w = (torch.randn(n, k, generator=g) * 0.05).bfloat16().to(DEV)
            wf = fragment_major(w)
            if gated:
                out = torch.full((m, n // 2), float("nan"), device=DEV, dtype=torch.bfloat16)
                lib.gemm_bf16(a, wf, out, 1, w_frag=True)
                wr = w.float().view(n // 32, 2, 16, k)
                want = torch.nn.functional.silu(a.float() @ wr[:, 0].reshape(n // 2, k).T) * (a.float() @ wr[:, 1].reshape(n // 2, k).T)
                assert _rel(out, want) < 1e-2, (units, m, n, k)
            else:
                terms = lib.gemm_bf16_terms(a, wf, w_frag=True)
                assert _rel(terms.sum(0), a.float() @ w.float().T) < 2e-3, (units, m, n, k, terms.shape[0])
    finally:
        lib._lib.rb_tune_compute_units(0)


@pytest.mark.parametrize("cfg", [4, 5, 6, 7, 8, 9, 10, 13])
def test_every_tile_of_the_direct_to_lds_product_at_sizes_that_fill_none(lib, cfg):
    """The planner picks a tile by the product's sizes, so sizes of a test reach only some of the
    tiles: here each is forced in turn (the hook that measurements use), with 1, 2 and 4 K slices,
    for token and row counts that fill no tile (rows a multiple of 16 only, as fragment-major W
    asks), W as rows and fragment-major, plain and gated."""
    from helpers import fragment_major
    k = 1024
    try:
        for m, n in ((33, 992), (200, 592), (300, 1376)):
            g = torch.Generator().manual_seed(cfg * 1000 + m)
            a = torch.randn(m, k, generator=g).bfloat16().to(DEV)
            w = (torch.randn(n, k, generator=g) * 0.05).bfloat16().to(DEV)
            wf = fragment_major(w)
            want = a.float() @ w.float().T
            for parts in (1, 2, 4):
                lib._lib.rb_tune_tiles(cfg, parts)
                terms = lib.gemm_bf16_terms(a, wf, w_frag=True)
                assert terms.shape == (parts, m, n), (cfg, parts, tuple(terms.shape))
                assert _rel(terms.sum(0), want) < 2e-3, (cfg, m, n, parts)
                assert torch.equal(lib.gemm_bf16_terms(a, w), terms), (cfg, m, n, parts)
            lib._lib.rb_tune_tiles(cfg, 1)
            if n % 32 == 0:
                out = torch.full((m, n // 2), float("nan"), device=DEV, dtype=torch.bfloat16)
                lib.gemm_bf16(a, wf, out, 1, w_frag=True)
                wr = w.float().view(n // 32, 2, 16, k)
                gate = a.float() @ wr[:, 0].reshape(n // 2, k).T
                up = a.float() @ wr[:, 1].reshape(n // 2, k).T
                assert _rel(out, torch.nn.functional.silu(gate) * up) < 1e-2, (cfg, m, n)
    finally:
        lib._lib.rb_tune_tiles(0, 0)


def test_gemm_bf16_few_refuses_other_sizes(lib):
    from rbitnet_amd.errors import KernelError
    assert not lib.gemm_bf16_few_ok(17, 64, 64)
    assert not lib.gemm_bf16_few_ok(4, 64, 60)
    a = torch.zeros(17, 64, device=DEV, dtype=torch.bfloat16)
    w = torch.zeros(64, 64, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(KernelError, match="not for it"):
        lib.gemm_bf16_few(a, w, torch.zeros(17, 64, device=DEV), 0)


def test_attention_long_context(lib):
    """Thousands of keys over many pages: decode with several split counts and a prompt step
    on top of a long past (chunked prefill), against the plain computation."""
    n_heads, n_kv, d = 8, 2, 128
    dtype = torch.bfloat16
    past, q_lens = [5000, 4097], [1, 1]
    g, bt, tok_seq, tok_pos, total = _paged_setup(past, q_lens, n_kv, d, dtype, n_pages=160, seed=9)
    k_full = [torch.randn(n, n_kv, d, generator=g).to(dtype) for n in total]
    v_full = [torch.randn(n, n_kv, d, generator=g).to(dtype) for n in total]
    q = (torch.randn(2, n_heads, d, generator=g) * 1.5).to(dtype)
    kp, vp = _fill_pages(k_full, v_full, bt, 160, n_kv, d, dtype)
    kp, vp = kp.to(DEV), vp.to(DEV)
    scale = 1 / math.sqrt(d)
    want = _attention_ref(q, k_full, v_full, tok_seq, tok_pos, n_heads, n_kv, scale, 0)
    for n_splits, mode in ((1, 0), (3, 0), (16, 0), (1, 1), (5, 1), (16, 1)):
        out = torch.full((2, n_heads * d), float("nan"), dtype=dtype, device=DEV)
        ws = torch.empty(2 * n_heads * n_splits * (d + 2), device=DEV)
        lib._lib.rb_tune_decode_mfma(mode)             # 1: the matrix-core kernel
        try:
            lib.attention_decode_bf16(q.to(DEV), kp, vp, out, tok_pos.to(DEV), bt.to(DEV), n_heads, n_kv, d, scale,
                                      0, n_splits, ws)
        finally:
            lib._lib.rb_tune_decode_mfma(0)
        assert _rel(out, want) < 1e-2, (n_splits, mode)
    # a 100-token step on top of 4000 cached tokens
    past, q_lens = [4000], [100]
    g, bt, tok_seq, tok_pos, total = _paged_setup(past, q_lens, n_kv, d, dtype, n_pages=160, seed=10)
    k_full = [torch.randn(n, n_kv, d, generator=g).to(dtype) for n in total]
    v_full = [torch.randn(n, n_kv, d, generator=g).to(dtype) for n in total]
    q = (torch.randn(100, n_heads, d, generator=g) * 1.5).to(dtype)
    kp, vp = _fill_pages(k_full, v_full, bt, 160, n_kv, d, dtype)
    out = torch.full((100, n_heads * d), float("nan"), dtype=dtype, device=DEV)
    cu = torch.tensor([0, 100], dtype=torch.int32, device=DEV)
    lib.attention_prefill_bf16(q.to(DEV), kp.to(DEV), vp.to(DEV), out, cu,
                               torch.tensor(past, dtype=torch.int32, device=DEV), bt.to(DEV), 1, 100, n_heads, n_kv,
                               d, scale, 0)
    want = _attention_ref(q, k_full, v_full, tok_seq, tok_pos, n_heads, n_kv, scale, 0)
    assert _rel(out, want) < 1.5e-2


def test_sample_frequencies_follow_softmax(lib):
    """20,000 draws with evenly spread uniform numbers: the frequency of every token is its
    softmax probability at the given temperature (to within a draw or two)."""
    g = torch.Generator().manual_seed(4)
    vocab, n, temp = 50, 20000, 0.7
    row = torch.randn(vocab, generator=g) * 2
    logits = row[None, :].expand(n, vocab).contiguous().to(DEV)
    us = ((torch.arange(n) + 0.5) / n).float().to(DEV)
    temps = torch.full((n,), temp, device=DEV)
    tokens = torch.empty(n, dtype=torch.int32, device=DEV)
    lib.sample(logits, temps, us, tokens)
    counts = torch.bincount(tokens.long().cpu(), minlength=vocab).double()
    want = torch.softmax(row.double() / temp, 0) * n
    assert float((counts - want).abs().max()) <= 2.0


# ------------------------------------------------------------------------ probes
def test_probes_read_every_byte_and_write_nothing(lib):
    """The streaming-read probes of the benchmark, in both modes: a lane whose values xor to a
    magic number raises the sink, so a buffer of zeros with that number in one place shows
    whether the place was read: the first and the last 16 bytes, one in the middle, one in the
    rest that is no whole piece of 64 KB.  They write nothing else and refuse a buffer they
    cannot read with 16-byte loads."""
    from rbitnet_amd.errors import KernelError
    magic = 0x9E3779B9 - (1 << 32)
    n = (3 << 20) // 4 + 4 * 1000                # three pieces of 64 KB x 16 and a rest, in int32 words
    for pieces in (False, True):
        for blocks in (1, 7, 64):
            for word in (0, n // 2 // 4 * 4, n - 4 * 500, n - 4):
                buf = torch.zeros(n, dtype=torch.int32, device=DEV)
                buf[word] = magic
                before = buf.clone()
                sink = torch.zeros(1, device=DEV)
                lib.probe_read(buf, sink, blocks, pieces)
                torch.cuda.synchronize()
                assert float(sink) == 1.0, (pieces, blocks, word)
                assert torch.equal(buf, before)
            sink = torch.zeros(1, device=DEV)
            lib.probe_read(torch.zeros(n, dtype=torch.int32, device=DEV), sink, blocks, pieces)
            torch.cuda.synchronize()
            assert float(sink) == 0.0
    sink = torch.zeros(1, device=DEV)
    assert lib.probe_mfma(8, 10, sink) == 8 * 10 * 4 * 2 * 32 * 32 * 16
    torch.cuda.synchronize()
    assert float(sink) == 0.0
    with pytest.raises(KernelError):
        lib.probe_read(torch.zeros(16, dtype=torch.int32, device=DEV)[:3], sink)


@pytest.mark.parametrize("m", [1, 5, 16, 17, 40, 64, 100, 256, 700, 2100])
@pytest.mark.parametrize("n,k,epi", [(4096, 1024, 0), (1008, 64, 0), (48, 128, 0), (6144, 4096, 0), (12288, 448, 0),
                                     (672, 256, 1), (8208 * 2, 384, 1), (28672, 512, 1)])
def test_gemm_bf16_with_w_stored_fragment_major(lib, m, n, k, epi):
    """Every matrix-core product kernel (tokens in registers, W streamed; tiles through LDS, with and
    without K slices) reads W in either layout and gives the same numbers bit for bit: the layout
    changes where a value lies, not which values a sum adds in which order."""
    from helpers import fragment_major
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).bfloat16().to(DEV)
    w = (torch.randn(n, k, generator=g) * 0.3).bfloat16()
    rows, frag = w.to(DEV), fragment_major(w).to(DEV)
    # the packing kernel writes the same layout
    packed = torch.full((n, k), float("nan"), dtype=torch.bfloat16, device=DEV)
    lib.place_rows(rows, packed, frag=True)
    assert torch.equal(packed, frag)
    shape = (m, n // 2 if epi else n)
    for dtype in (torch.float32, torch.bfloat16):
        want = torch.full(shape, float("nan"), device=DEV, dtype=dtype)
        got = torch.full(shape, float("nan"), device=DEV, dtype=dtype)
        lib.gemm_bf16(a, rows, want, epi)
        lib.gemm_bf16(a, frag, got, epi, w_frag=True)
        assert torch.equal(got, want), float((got.float() - want.float()).abs().max())
    if not epi:
        assert torch.equal(lib.gemm_bf16_terms(a, frag, w_frag=True), lib.gemm_bf16_terms(a, rows))
        oracle = a.double().cpu() @ w.double().T
        assert _rel(want.float(), oracle) < 1e-2
    if m <= 16 and not epi and lib.gemm_bf16_few_ok(m, n, k):
        for epilogue in (2, 3):
            outs = []
            for mat, is_frag in ((rows, False), (frag, True)):
                c = torch.ones((m, n), device=DEV)
                gain = torch.linspace(0.5, 1.5, n, device=DEV)
                gained = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
                squares = torch.empty((m, (n + 15) // 16), device=DEV)
                lib.gemm_bf16_few(a, mat, c, epilogue, gain=gain, gained=gained, squares_out=squares, w_frag=is_frag)
                outs.append((c, gained, squares) if epilogue == 3 else (c,))
            for x, y in zip(*outs):
                assert torch.equal(x, y)


def test_fragment_major_refuses_sizes_it_is_not_for(lib):
    from rbitnet_amd.errors import KernelError
    a = torch.zeros(4, 72, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(32, 72, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(KernelError, match="fragment-major"):
        lib.gemm_bf16(a, w, torch.empty(4, 32, device=DEV), 0, w_frag=True)
    with pytest.raises(KernelError, match="layout"):
        lib.place_rows(torch.zeros(8, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(8, 64, dtype=torch.bfloat16, device=DEV), frag=True)
