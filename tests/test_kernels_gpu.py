"""Each HIP kernel alone against a plain float32 torch computation of the same op,
at sizes other than the engine's: widths and vocabularies that are no power of two,
head sizes in steps of 16, odd head and group counts, page edges."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype, f32=1e-5, bf16=2e-2):
    return dict(rtol=f32, atol=f32) if dtype == torch.float32 else dict(rtol=bf16, atol=bf16)


@pytest.fixture(scope="module")
def ops():
    from llm_runtime_study_amd.kernels import ops as _ops

    _ops.library()
    return _ops


@pytest.fixture
def all_rows_in_own_kernel(ops):
    """The few-rows kernel takes up to 64 rows; in steps callers hand over to other kernels from 17 rows
    on.  The choice that lifts that, for tests of the kernel itself (passed with the call: nothing is set
    in the library)."""
    return ops.KernelChoice(few_rows_max=ops.few_rows_capacity())


def dev(t):
    return t.to("cuda")


def close_in_norm(got, want, rel=1e-2):
    """bfloat16 results of long sums: the error is a small part of the whole (relative L2 norm) and
    no single element strays by more than a few units of the largest one's rounding."""
    got, want = got.cpu().double(), want.double()
    assert (got - want).norm() <= rel * want.norm(), f"relative error {(got - want).norm() / want.norm():.3g}"
    assert (got - want).abs().max() <= 2e-2 * want.abs().max() + 2e-2, f"largest error {(got - want).abs().max():.3g}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,hidden,vocab", [(1, 64, 256), (7, 96, 331), (33, 4096, 1000)])
def test_embed(ops, dtype, tokens, hidden, vocab):
    g = torch.Generator().manual_seed(0)
    table = torch.randn(vocab, hidden, generator=g).to(dtype)
    ids = torch.randint(0, vocab, (tokens,), generator=g, dtype=torch.int32)
    ids[0] = vocab - 1
    out = torch.empty(tokens, hidden, device="cuda")
    ops.embed(out, dev(table), dev(ids))
    torch.testing.assert_close(out.cpu(), table.float()[ids.long()], rtol=0, atol=0)


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("rows,hidden,eps", [(1, 64, 1e-6), (5, 96, 1e-5), (3, 4096, 1e-6), (2, 5120 + 16, 1e-3)])
def test_rmsnorm(ops, out_dtype, w_dtype, rows, hidden, eps):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(rows + 2, hidden, generator=g) * 3
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(w_dtype)
    want = w.float() * (x * torch.rsqrt(x.square().mean(-1, keepdim=True) + eps))
    out = torch.empty(rows, hidden, device="cuda", dtype=out_dtype)
    ops.rmsnorm(out, dev(x), dev(w), eps)
    torch.testing.assert_close(out.cpu().float(), want[:rows], **tol(out_dtype, 2e-6, 1e-2))
    pick = torch.tensor([rows + 1, 0, rows][:rows] + [1] * max(0, rows - 3), dtype=torch.int32)
    ops.rmsnorm(out, dev(x), dev(w), eps, rows=dev(pick))
    torch.testing.assert_close(out.cpu().float(), want[pick.long()], **tol(out_dtype, 2e-6, 1e-2))


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("rows,hidden,eps", [(1, 64, 1e-6), (33, 96, 1e-5), (300, 4096, 1e-6), (2, 5120 + 16, 1e-3), (3, 9000, 1e-5), (4, 50, 1e-5)])
def test_add_rmsnorm(ops, out_dtype, rows, hidden, eps):
    """The residual add and the norm after it in one kernel: the stream is updated in place and
    the norm is that of the updated rows."""
    g = torch.Generator().manual_seed(rows + hidden)
    x = torch.randn(rows, hidden, generator=g) * 3
    y = torch.randn(rows, hidden, generator=g).bfloat16()
    w = (1 + 0.2 * torch.randn(hidden, generator=g)).bfloat16()
    stream = dev(x.clone())
    out = torch.empty(rows, hidden, device="cuda", dtype=out_dtype)
    ops.add_rmsnorm(out, stream, dev(y), dev(w), eps)
    want_stream = x + y.float()
    torch.testing.assert_close(stream.cpu(), want_stream, rtol=0, atol=0)
    want = w.float() * want_stream * torch.rsqrt(want_stream.pow(2).mean(-1, keepdim=True) + eps)
    torch.testing.assert_close(out.cpu().float(), want, **tol(out_dtype, 1e-5, 1e-2))


@pytest.mark.parametrize("hidden", [64, 4096])
def test_every_norm_kernel_has_eps_under_the_square_root(ops, hidden):
    """eps = 0.5 beside a mean of squares of 0.25: x * rsqrt(mean + eps) is x / 0.866, while x / (sqrt(mean) + eps)
    would be x / 1.0.  The norm kernel, the add-and-norm kernel, the norm folded into a product's input, and the
    norm taken apart around products of few rows and of 17..128 rows."""
    g = torch.Generator().manual_seed(hidden)
    rows, eps = 3, 0.5
    x = 0.5 * torch.sign(torch.randn(rows, hidden, generator=g))
    w = (1 + 0.25 * torch.randn(hidden, generator=g)).bfloat16()
    want = w.float() * x / math.sqrt(0.75)
    assert ((want - w.float() * x).abs() / want.abs()).min() > 0.13          # the misreading is 13 % away, the tolerances below 1-2 %
    for out_dtype in DTYPES:
        out = torch.empty(rows, hidden, device="cuda", dtype=out_dtype)
        ops.rmsnorm(out, dev(x), dev(w), eps)
        torch.testing.assert_close(out.cpu().float(), want, **tol(out_dtype, 2e-6, 1e-2))
        stream = dev(x - 1.0)
        ops.add_rmsnorm(out, stream, dev(torch.ones(rows, hidden).bfloat16()), dev(w), eps)
        torch.testing.assert_close(out.cpu().float(), want, **tol(out_dtype, 2e-6, 1e-2))
    # folded into a product's input: the product with the identity gives the normalised rows back
    eye = torch.eye(hidden).bfloat16()
    out = torch.empty(rows, hidden, device="cuda", dtype=torch.float32)
    ops.gemm(out, dev(x), dev(eye), norm_weight=dev(w), eps=eps)
    torch.testing.assert_close(out.cpu(), want, rtol=1e-2, atol=1e-2)
    # taken apart: a product that adds zero into the stream begins the norm, scale_rows or the next product finishes it
    for m in (rows, 24):
        if m > 16 and hidden % 256:
            continue
        xs = x[torch.arange(m) % rows]
        stream = dev(xs.clone())
        zeros_a, zeros_w = torch.zeros(m, hidden, dtype=torch.bfloat16, device="cuda"), torch.zeros(hidden, hidden, dtype=torch.bfloat16, device="cuda")
        next_x = torch.empty(m, hidden, dtype=torch.bfloat16, device="cuda")
        if m <= 16:
            sumsq = torch.empty(ops.norm_chain_parts(hidden), m, device="cuda")
            ops.gemm_norm_chain(stream, zeros_a, zeros_w, accumulate=True, next_x=next_x, next_sumsq=sumsq, next_weight=dev(w))
        else:
            sumsq = torch.empty(ops.norm_begin_parts(hidden), m, device="cuda")
            ops.gemm_mid_add_norm_begin(stream, zeros_a, zeros_w, dev(w), next_x, sumsq)
        finished = torch.empty(m, hidden, dtype=torch.bfloat16, device="cuda")
        ops.scale_rows(finished, next_x, sumsq, eps)
        torch.testing.assert_close(finished.cpu().float(), want[torch.arange(m) % rows], rtol=1e-2, atol=1e-2)
        out = torch.empty(m, hidden, dtype=torch.float32, device="cuda")
        if m <= 16:
            ops.gemm_norm_chain(out, next_x, dev(eye), in_sumsq=sumsq, in_eps=eps)
        else:
            ops.gemm_mid_scaled(out, next_x, dev(eye), sumsq, eps)
        torch.testing.assert_close(out.cpu(), want[torch.arange(m) % rows], rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("half,theta", [(8, 1e4), (16, 1e6), (64, 1e6), (24, 5e5)])
def test_rope_table(ops, half, theta):
    positions = torch.tensor([0, 1, 2, 17, 511, 4095, 40959], dtype=torch.int32)
    inv = 1.0 / (theta ** (torch.arange(0, 2 * half, 2, dtype=torch.float32) / (2 * half)))
    cos = torch.empty(len(positions), half, device="cuda")
    sin = torch.empty_like(cos)
    ops.rope_table(cos, sin, dev(positions), dev(inv))
    angles = positions.float().unsqueeze(-1) * inv
    torch.testing.assert_close(cos.cpu(), angles.cos(), rtol=0, atol=2e-7)
    torch.testing.assert_close(sin.cpu(), angles.sin(), rtol=0, atol=2e-7)
    # against float64 angles: what float32 tables can give at position 40959
    exact = (positions.double().unsqueeze(-1) * inv.double()).cos()
    assert (cos.cpu().double() - exact).abs().max() < 3e-3


def _qk_prep_reference(qkv, nq, nkv, d, qw, kw, eps, positions, inv, rot_half):
    t = qkv.shape[0]
    heads = qkv.float().view(t, nq + 2 * nkv, d)
    q, k, v = heads[:, :nq], heads[:, nq:nq + nkv], heads[:, nq + nkv:]

    def norm(x, w):
        if w is None:
            return x
        return w.float() * (x * torch.rsqrt(x.square().mean(-1, keepdim=True) + eps))

    def rotate(x):
        if rot_half == 0:
            return x
        ang = positions.float().view(t, 1, 1) * inv.view(1, 1, -1)
        c, s = ang.cos(), ang.sin()
        a, b, rest = x[..., :rot_half], x[..., rot_half:2 * rot_half], x[..., 2 * rot_half:]
        return torch.cat((a * c - b * s, b * c + a * s, rest), -1)

    return rotate(norm(q, qw)), rotate(norm(k, kw)), v


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layout", ["scattered", "runs"])
@pytest.mark.parametrize("nq,nkv,d,rot,normed,page", [
    (4, 2, 16, 16, True, 4), (8, 2, 32, 32, True, 16), (3, 3, 48, 32, False, 8),
    (32, 8, 128, 128, True, 16), (5, 1, 80, 0, True, 16), (6, 2, 256, 256, True, 64),
])
def test_qk_prep(ops, dtype, layout, nq, nkv, d, rot, normed, page):
    """A few tokens with slots anywhere; and a step of many tokens (which stores the values through
    a kernel of its own) whose requests occupy runs of slots that start and end inside pages."""
    g = torch.Generator().manual_seed(2)
    if layout == "scattered":
        t, pages = 19, 12
        slots = torch.randperm(pages * page, generator=g)[:t].to(torch.int32)
    else:
        runs, at, pieces = [1, 7, 16, 33, 64, 100, 79, 5], 3, []
        for n in runs:                                   # each request starts somewhere inside a fresh page
            pieces.append(torch.arange(at, at + n))
            at = -(-(at + n) // page) * page + page + int(torch.randint(0, page, (1,), generator=g))
        order = torch.randperm(len(pieces), generator=g).tolist()
        slots = torch.cat([pieces[i] for i in order]).to(torch.int32)
        t, pages = slots.numel(), -(-at // page) + 1
    slots[3] = -1  # a token that must not be stored
    qkv = torch.randn(t, (nq + 2 * nkv) * d, generator=g).to(dtype)
    qw = (1 + 0.1 * torch.randn(d, generator=g)).to(dtype) if normed else None
    kw = (1 + 0.1 * torch.randn(d, generator=g)).to(dtype) if normed else None
    positions = torch.randint(0, 3000, (t,), generator=g, dtype=torch.int32)
    rot_half = rot // 2
    inv = 1.0 / (1e4 ** (torch.arange(0, rot, 2, dtype=torch.float32) / max(rot, 1)))
    want_q, want_k, want_v = _qk_prep_reference(qkv, nq, nkv, d, qw, kw, 1e-6, positions, inv, rot_half)

    d_qkv = dev(qkv)
    kp = torch.full((pages, nkv, page, d), 7.0, device="cuda", dtype=dtype)
    vp = torch.full((pages, nkv, d, page), 7.0, device="cuda", dtype=dtype)   # values: transposed inside a page
    cos = sin = None
    if rot_half:
        cos = torch.empty(t, rot_half, device="cuda")
        sin = torch.empty_like(cos)
        ops.rope_table(cos, sin, dev(positions), dev(inv))
    ops.qk_prep(d_qkv, nq, nkv, d, None if qw is None else dev(qw), None if kw is None else dev(kw), 1e-6,
                cos, sin, kp, vp, dev(slots), page)
    got = d_qkv.cpu().float().view(t, nq + 2 * nkv, d)
    torch.testing.assert_close(got[:, :nq], want_q, **tol(dtype, 1e-5, 2e-2))
    kp, vp = kp.cpu().float(), vp.cpu().float()
    touched = torch.zeros(pages, page, dtype=torch.bool)
    for i in range(t):
        s = int(slots[i])
        if s < 0:
            continue
        touched[s // page, s % page] = True
        torch.testing.assert_close(kp[s // page, :, s % page], want_k[i], **tol(dtype, 1e-5, 2e-2))
        torch.testing.assert_close(vp[s // page, :, :, s % page], want_v[i], rtol=0, atol=0)
    # nothing else was written
    assert (kp.permute(0, 2, 1, 3)[~touched] == 7.0).all() and (vp.permute(0, 3, 1, 2)[~touched] == 7.0).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,inter", [(1, 128), (9, 160), (4, 12288), (300, 331)])
def test_silu_mul(ops, dtype, tokens, inter):
    g = torch.Generator().manual_seed(3)
    gu = (torch.randn(tokens, 2 * inter, generator=g) * 2).to(dtype)
    out = torch.empty(tokens, inter, device="cuda", dtype=dtype)
    ops.silu_mul(out, dev(gu))
    gate, up = gu.float()[:, :inter], gu.float()[:, inter:]
    torch.testing.assert_close(out.cpu().float(), torch.nn.functional.silu(gate) * up, **tol(dtype, 1e-6, 1e-2))
    if inter % 8 == 0:   # groups of 8 gate columns followed by their 8 up columns
        mixed = torch.stack((gu[:, :inter].view(tokens, inter // 8, 8), gu[:, inter:].view(tokens, inter // 8, 8)), 2).reshape(tokens, 2 * inter)
        ops.silu_mul(out, dev(mixed.contiguous()), interleaved=True)
        torch.testing.assert_close(out.cpu().float(), torch.nn.functional.silu(gate) * up, **tol(dtype, 1e-6, 1e-2))


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_into(ops, dtype):
    g = torch.Generator().manual_seed(13)
    residual = torch.randn(37, 331, generator=g)
    y = torch.randn(37, 331, generator=g).to(dtype)
    out = dev(residual.clone())
    ops.add_into(out, dev(y))
    torch.testing.assert_close(out.cpu(), residual + y.float(), rtol=0, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [
    (1, 64, 64), (5, 331, 96), (17, 160, 96), (64, 256, 160), (130, 200, 264), (3, 129, 40),
    (2, 70, 36), (1, 1000, 4096), (257, 384, 512),
    (8, 5120, 160), (3, 4112, 72), (16, 12290, 64),      # few rows, widths that are dealt out unevenly by 16-row tiles
    (300, 516, 96), (1100, 4096, 1024),                  # many rows, K a multiple of 32: the kernel of 128 x 256 tiles, ragged edges and 8 XCDs' numbering
    (2000, 16648, 192), (2048, 16384, 64),               # many rows and wide, K a multiple of 64: the kernel of 256 x 256 tiles, ragged edges
    (2000, 4232, 192), (2048, 4096, 64),                 # ... and less wide: its form of 256 x 128 tiles
    (2000, 6100, 192), (2048, 6144, 64),                 # ... and 256 tiles of 256 x 192
    (512, 4096, 2048), (520, 4232, 2048), (300, 9000, 1088),   # too few 256 x 128 tiles for the chip: K divided between workgroups (4, 2 and 1 parts)
])
@pytest.mark.parametrize("mode", ["store", "store_f32", "add"])
def test_gemm(ops, dtype, m, n, k, mode):
    g = torch.Generator().manual_seed(4)
    a = torch.randn(m, k, generator=g).to(dtype)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(dtype)
    bias = torch.randn(n, generator=g).to(dtype) if n % 2 else None
    want = a.double() @ w.double().T + (0 if bias is None else bias.double())
    if mode == "store":
        out = torch.empty(m, n, device="cuda", dtype=dtype)
    else:
        out = torch.full((m, n), 0.5, device="cuda")
    ops.gemm(out, dev(a), dev(w), None if bias is None else dev(bias), accumulate=(mode == "add"))
    if mode == "add":
        want = want + 0.5
    if dtype == torch.float32:
        torch.testing.assert_close(out.cpu().double(), want, rtol=1e-5, atol=1e-5)
    elif mode == "store":
        torch.testing.assert_close(out.cpu().double(), want, rtol=1e-2, atol=1e-2)
    else:  # bf16 inputs, float32 accumulation and output: only the summation order differs
        torch.testing.assert_close(out.cpu().double(), want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("m", [17, 32, 40, 48, 49, 64, 65, 96, 100, 128])
@pytest.mark.parametrize("n,k", [(64, 256), (208, 512), (4096, 1024), (6144, 4096), (1040, 3328)])
@pytest.mark.parametrize("waves,splits", [(0, 0), (4, 1), (5, 1), (5, 3), (6, 2), (8, 3), (4, 8)])
def test_gemm_of_17_to_64_rows(ops, m, n, k, waves, splits):
    """The kernel for 17..64 rows (K a multiple of 256): every workgroup shape, K divided between
    workgroups or not, ragged last tiles, all three output modes and the gated epilogue."""
    g = torch.Generator().manual_seed(m * 131 + n + k)
    a = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).bfloat16()
    want = a.double() @ w.double().T
    choice = ops.KernelChoice(mid_waves=waves, mid_splits=splits)
    stored = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
    ops.gemm(stored, dev(a), dev(w), choice=choice)
    wide = torch.full((m, n), 0.5, device="cuda")
    ops.gemm(wide, dev(a), dev(w), accumulate=True, choice=choice)
    plain = torch.empty(m, n, device="cuda")
    ops.gemm(plain, dev(a), dev(w), choice=choice)
    inter = n // 2
    gate, up = w[:inter], w[inter:]
    mixed = torch.stack((gate.view(inter // 8, 8, k), up.view(inter // 8, 8, k)), 1).reshape(n, k).contiguous()
    gated = torch.empty(m, inter, device="cuda", dtype=torch.bfloat16)
    ops.gemm(gated, dev(a), dev(mixed), swiglu=True, choice=choice)
    torch.testing.assert_close(stored.cpu().double(), want, rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(plain.cpu().double(), want, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(wide.cpu().double(), want + 0.5, rtol=1e-4, atol=1e-4)
    close_in_norm(gated, torch.nn.functional.silu(want[:, :inter]) * want[:, inter:])


@pytest.mark.parametrize("m", [17, 33, 48, 64])
@pytest.mark.parametrize("n,k,deal", [(17984, 512, (4, 256, 100)), (36848, 256, (8, 256, 255)), (37568, 768, (4, 512, 300)), (17976, 512, (4, 256, 100)),
                                      (34816, 1024, (8, 256, 128)), (25808, 512, (6, 256, 77)), (51200, 256, (6, 512, 128))])
def test_gemm_of_17_to_64_rows_with_rows_dealt_evenly(ops, m, n, k, deal):
    """The kernel for 17..64 rows with its weight rows dealt out over a whole multiple of the compute units, some
    workgroups with a tile more than their waves (the extra tile's k steps go round the waves and meet in LDS): every
    output mode, the gated epilogue, a norm begun before, a ragged last tile; and the same results as the plain deal."""
    if ops.compute_units() != 256:
        pytest.skip("the shapes are made for 256 compute units")
    even, plain_deal = ops.KernelChoice(mid_even=2), ops.KernelChoice(mid_even=1)
    assert ops.gemm_mid_deal(m, n, k, even) == (deal[0], 1, deal[1], deal[2])
    assert ops.gemm_mid_deal(m, n, k, plain_deal)[3] == 0
    g = torch.Generator().manual_seed(m * 7 + n + k)
    a = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).bfloat16()
    want = a.double() @ w.double().T
    sumsq = torch.rand(3, m, generator=g) * k
    results = {}
    for name, choice in (("even", even), ("plain", plain_deal)):
        stored = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
        ops.gemm(stored, dev(a), dev(w), choice=choice)
        wide = torch.full((m, n), 0.5, device="cuda")
        ops.gemm(wide, dev(a), dev(w), accumulate=True, choice=choice)
        plain = torch.empty(m, n, device="cuda")
        ops.gemm(plain, dev(a), dev(w), choice=choice)
        torch.testing.assert_close(stored.cpu().double(), want, rtol=1e-2, atol=1e-2)
        torch.testing.assert_close(plain.cpu().double(), want, rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(wide.cpu().double(), want + 0.5, rtol=1e-4, atol=1e-4)
        results[name] = [stored.cpu(), plain.cpu()]
        if n % 16 == 0:
            inter = n // 2
            mixed = torch.stack((w[:inter].view(inter // 8, 8, k), w[inter:].view(inter // 8, 8, k)), 1).reshape(n, k).contiguous()
            gated = torch.empty(m, inter, device="cuda", dtype=torch.bfloat16)
            ops.gemm(gated, dev(a), dev(mixed), swiglu=True, choice=choice)
            close_in_norm(gated, torch.nn.functional.silu(want[:, :inter]) * want[:, inter:])
            # behind a norm that the product before began: rows scaled by the factor of their partial sums of squares
            eps = 1e-5
            factor = torch.rsqrt(sumsq.double().sum(0) / k + eps)[:, None]
            scaled = torch.empty(m, inter, device="cuda", dtype=torch.bfloat16)
            ops.gemm_mid_scaled(scaled, dev(a), dev(mixed), dev(sumsq), eps, swiglu=True, choice=choice)
            y = want * factor
            close_in_norm(scaled, torch.nn.functional.silu(y[:, :inter]) * y[:, inter:], 1e-2)
            results[name] += [gated.cpu(), scaled.cpu()]
    # the sums of a column are added in the same order of k either way (slices in turn, steps in turn) only within a
    # wave; the extra tile's are added wave by wave, so its columns may differ in the last bit of the float32 sum
    for one, other in zip(results["even"], results["plain"]):
        torch.testing.assert_close(one.double(), other.double(), rtol=1e-2 if one.dtype == torch.bfloat16 else 1e-5, atol=1e-2 if one.dtype == torch.bfloat16 else 1e-5)


@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(512, 4096, 4096), (300, 1024, 3072), (257, 7000, 1088), (129, 512, 8192)])
def test_product_of_many_rows_with_residual_add_and_norm_in_its_finishing_kernel(ops, w_dtype, m, n, k):
    """residual += a w^T and the RMSNorm of the result in two kernels (K divided between workgroups or the tiles as
    they are; the kernel that adds up the sums adds the residual and normalises), with the caller's own workspace and
    with the one the process keeps: the same bits, and both as the plain computation."""
    if ops.gemm_lines_splits(m, n, k) < 1:
        pytest.skip("the divided product does not take this shape on this device")
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).bfloat16()
    res = torch.randn(m, n, generator=g)
    nw = (1 + 0.1 * torch.randn(n, generator=g)).to(w_dtype)
    eps = 1e-5
    want_res = res.double() + a.double() @ w.double().T
    want = nw.double() * want_res * torch.rsqrt(want_res.square().mean(-1, keepdim=True) + eps)
    outs = []
    for own in (True, False):
        residual = dev(res.clone())
        normed = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
        space = torch.empty(ops.gemm_workspace_bytes() // 4, device="cuda") if own else None
        ops.gemm_lines_add_rmsnorm(residual, dev(a), dev(w), dev(nw), eps, normed, workspace=space)
        torch.testing.assert_close(residual.cpu().double(), want_res, rtol=1e-4, atol=1e-4)
        close_in_norm(normed, want, rel=5e-3)
        outs.append((residual.cpu(), normed.cpu()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    # the same product through gemm() and the norm kernel: the residual stream bit for bit
    residual = dev(res.clone())
    ops.gemm(residual, dev(a), dev(w), accumulate=True)
    assert torch.equal(residual.cpu(), outs[0][0])
    with pytest.raises(Exception, match="workspace"):
        ops.gemm(residual, dev(a), dev(w), accumulate=True, workspace=torch.empty(1024, device="cuda"))


@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("m,h,n2,k,swiglu,splits", [(17, 256, 64, 256, False, 0), (40, 512, 208, 1024, True, 2), (64, 4096, 6144, 4096, False, 0),
                                                     (100, 1024, 2048, 3328, True, 3), (128, 4096, 24576, 512, True, 0)])
def test_gemm_of_17_to_128_rows_with_norm_taken_apart(ops, w_dtype, m, h, n2, k, swiglu, splits):
    """residual += x W1^T begins the RMSNorm of the new residual (bf16(h * weight) and partial sums of squares, left by
    the kernel that adds the K splits' sums); the next product finishes it in its epilogue, or scale_rows does."""
    g = torch.Generator().manual_seed(m + h + n2 + k)
    a = torch.randn(m, k, generator=g).bfloat16()
    w1 = (torch.randn(h, k, generator=g) / math.sqrt(k)).bfloat16()
    w2 = (torch.randn(n2, h, generator=g) / math.sqrt(h)).bfloat16()
    residual = torch.randn(m, h, generator=g) * 2
    gamma = (1 + 0.2 * torch.randn(h, generator=g)).to(w_dtype)
    eps = 1e-5
    updated = residual.double() + a.double() @ w1.double().T
    normed = gamma.double() * updated * torch.rsqrt(updated.square().mean(-1, keepdim=True) + eps)
    out = dev(residual.clone())
    next_x = torch.empty(m, h, device="cuda", dtype=torch.bfloat16)
    sumsq = torch.empty(ops.norm_begin_parts(h), m, device="cuda")
    choice = ops.KernelChoice(mid_splits=splits)
    ops.gemm_mid_add_norm_begin(out, dev(a), dev(w1), dev(gamma), next_x, sumsq, choice=choice)
    torch.testing.assert_close(out.cpu().double(), updated, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(sumsq.sum(0).cpu().double(), updated.square().sum(-1), rtol=1e-4, atol=1e-4)
    finished = torch.empty(m, h, device="cuda", dtype=torch.bfloat16)
    ops.scale_rows(finished, next_x, sumsq, eps)
    close_in_norm(finished, normed, 5e-3)
    if swiglu:
        inter = n2 // 2
        mixed = torch.stack((w2[:inter].view(inter // 8, 8, h), w2[inter:].view(inter // 8, 8, h)), 1).reshape(n2, h).contiguous()
        got = torch.empty(m, inter, device="cuda", dtype=torch.bfloat16)
        ops.gemm_mid_scaled(got, next_x, dev(mixed), sumsq, eps, swiglu=True, choice=choice)
        y = normed @ w2.double().T
        close_in_norm(got, torch.nn.functional.silu(y[:, :inter]) * y[:, inter:], 1e-2)
    else:
        got = torch.empty(m, n2, device="cuda")
        ops.gemm_mid_scaled(got, next_x, dev(w2), sumsq, eps, choice=choice)
        close_in_norm(got, normed @ w2.double().T, 5e-3)


@pytest.mark.parametrize("m,nq,nkv,d,k,splits,begun", [(17, 4, 2, 64, 256, 0, False), (64, 32, 8, 128, 4096, 0, True), (100, 6, 2, 32, 1024, 2, True),
                                                       (128, 8, 8, 128, 512, 1, False)])
def test_qkv_product_of_17_to_128_rows_with_head_preparation(ops, m, nq, nkv, d, k, splits, begun):
    """The q/k/v product whose K splits' sums are added up by the kernel that normalises and rotates the heads
    and writes k and v into the pages, against the product, qk_prep and the plain formulas one after the other."""
    g = torch.Generator().manual_seed(m + nq + d + k)
    n, page, pages = (nq + 2 * nkv) * d, 16, 12
    h = torch.randn(m, k, generator=g) * 2
    gamma = 1 + 0.2 * torch.randn(k, generator=g)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).bfloat16()
    qw, kw = (1 + 0.2 * torch.randn(d, generator=g)).bfloat16(), (1 + 0.2 * torch.randn(d, generator=g)).bfloat16()
    positions = torch.randint(0, 500, (m,), generator=g)
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, d, 2).float() / d))
    angle = positions.float()[:, None] * inv_freq[None, :]
    cos, sin = dev(angle.cos().contiguous()), dev(angle.sin().contiguous())
    slots = torch.randperm(pages * page, generator=g)[:m].to(torch.int32)
    eps, norm_eps = 1e-6, 1e-5
    if begun:     # the input is a norm begun before: x = bf16(h * gamma) and partial sums of h^2
        x = (h * gamma).bfloat16()
        parts = 3
        sumsq = torch.stack([h[:, i::parts].square().sum(-1) for i in range(parts)]).contiguous()
        source = x.double() * torch.rsqrt(h.double().square().mean(-1, keepdim=True) + norm_eps)
    else:
        x, sumsq = h.bfloat16(), None
        source = x.double()
    y = source @ w.double().T

    def rms(v, weight):
        return weight.double() * v * torch.rsqrt(v.square().mean(-1, keepdim=True) + eps)

    def rotate(v):
        c, s_ = angle.cos().double()[:, None, :], angle.sin().double()[:, None, :]
        a, b = v[..., : d // 2], v[..., d // 2:]
        return torch.cat((a * c - b * s_, b * c + a * s_), -1)

    q_want = rotate(rms(y[:, : nq * d].view(m, nq, d), qw))
    k_want = rotate(rms(y[:, nq * d: (nq + nkv) * d].view(m, nkv, d), kw))
    v_want = y[:, (nq + nkv) * d:].view(m, nkv, d)
    qkv = torch.zeros(m, n, device="cuda", dtype=torch.bfloat16)
    k_pages = torch.zeros(pages, nkv, page, d, device="cuda", dtype=torch.bfloat16)
    v_pages = torch.zeros(pages, nkv, d, page, device="cuda", dtype=torch.bfloat16)
    ops.gemm_mid_qk_prep(qkv, dev(x), dev(w), None if sumsq is None else dev(sumsq), norm_eps, nq, nkv, d, dev(qw), dev(kw), eps,
                         cos, sin, k_pages, v_pages, dev(slots), page, choice=ops.KernelChoice(mid_splits=splits))
    close_in_norm(qkv[:, : nq * d], q_want.reshape(m, nq * d), 1e-2)
    pg, off = (slots // page).long(), (slots % page).long()
    close_in_norm(k_pages.cpu()[pg, :, off, :], k_want, 1e-2)
    close_in_norm(v_pages.cpu()[pg, :, :, off], v_want, 1e-2)


@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 64, 96), (8, 331, 160), (17, 200, 96), (64, 6144, 4096), (33, 48, 264)])
def test_gemm_with_fused_rmsnorm_input(ops, w_dtype, m, n, k, all_rows_in_own_kernel):
    """The product of the RMSNorm of float32 rows, picked through a row list, in one kernel."""
    g = torch.Generator().manual_seed(14)
    h = torch.randn(m + 3, k, generator=g) * 4
    gamma = (1 + 0.2 * torch.randn(k, generator=g)).to(w_dtype)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).bfloat16()
    rows = torch.randperm(m + 3, generator=g)[:m].to(torch.int32)
    eps = 1e-5
    assert ops.gemm_fuses_norm(torch.bfloat16, m, k, all_rows_in_own_kernel) and ops.gemm_fuses_norm(torch.bfloat16, m, k) == (m <= 16)
    normed = gamma.double() * (h.double() * torch.rsqrt(h.double().square().mean(-1, keepdim=True) + eps))
    want = normed[rows.long()] @ w.double().T
    out = torch.empty(m, n, device="cuda")
    ops.gemm(out, dev(h), dev(w), norm_weight=dev(gamma), eps=eps, rows=dev(rows), count=m, choice=all_rows_in_own_kernel)
    close_in_norm(out, want, 5e-3)
    # without a row list the first m rows are taken; against the two-kernel path the only
    # difference is where the input is rounded to bfloat16
    x = torch.empty(m, k, device="cuda", dtype=torch.bfloat16)
    ops.rmsnorm(x, dev(h), dev(gamma), eps)
    two = torch.empty(m, n, device="cuda")
    ops.gemm(two, x, dev(w))
    ops.gemm(out, dev(h), dev(w), norm_weight=dev(gamma), eps=eps, choice=all_rows_in_own_kernel)
    close_in_norm(out, two.cpu(), 5e-3)


@pytest.mark.parametrize("m,inter,k", [(1, 128, 64), (9, 160, 96), (64, 12288, 4096), (65, 160, 96), (300, 136, 264),
                                       (300, 392, 160), (2048, 1024, 512),       # K a multiple of 32 and more than 64 rows: the kernel of 128 x 256 tiles
                                       (2040, 8200, 128), (2040, 2056, 128), (2040, 3072, 128),     # wide enough for the kernel of 256 x 256 tiles, for its 256 x 128 and its 256 x 192 form
                                       (500, 4104, 1024)])                       # K divided between workgroups of 256 x 128 tiles
def test_gemm_with_swiglu_epilogue(ops, m, inter, k, all_rows_in_own_kernel):
    """Gate and up rows interleaved in groups of 8; the product writes silu(gate) * up."""
    g = torch.Generator().manual_seed(15)
    x = torch.randn(m, k, generator=g).bfloat16()
    gate = (torch.randn(inter, k, generator=g) / math.sqrt(k) * 2).bfloat16()
    up = (torch.randn(inter, k, generator=g) / math.sqrt(k) * 2).bfloat16()
    mixed = torch.stack((gate.view(inter // 8, 8, k), up.view(inter // 8, 8, k)), 1).reshape(2 * inter, k).contiguous()
    want = torch.nn.functional.silu(x.double() @ gate.double().T) * (x.double() @ up.double().T)
    out = torch.empty(m, inter, device="cuda", dtype=torch.bfloat16)
    ops.gemm(out, dev(x), dev(mixed), swiglu=True)
    close_in_norm(out, want)
    if m <= 64:   # with the normalisation folded in as well
        h = torch.randn(m, k, generator=g) * 3
        gamma = (1 + 0.1 * torch.randn(k, generator=g)).bfloat16()
        xn = gamma.double() * (h.double() * torch.rsqrt(h.double().square().mean(-1, keepdim=True) + 1e-6))
        want = torch.nn.functional.silu(xn @ gate.double().T) * (xn @ up.double().T)
        ops.gemm(out, dev(h), dev(mixed), swiglu=True, norm_weight=dev(gamma), eps=1e-6, choice=all_rows_in_own_kernel)
        close_in_norm(out, want)


@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("m,h,n2,k,swiglu", [(1, 64, 96, 32, False), (8, 4096, 6144, 4096, False), (16, 4096, 24576, 12288, True),
                                             (5, 104, 328, 72, False), (9, 96, 320, 160, True), (3, 16400, 48, 64, False),
                                             (7, 5120, 7168, 640, False), (4, 4112, 4400, 96, False)])
def test_gemm_with_norm_taken_apart(ops, w_dtype, m, h, n2, k, swiglu):
    """Two products with an RMSNorm of the residual stream between them: the first adds into the
    stream and leaves bf16(h * weight) with partial sums of squares, the second finishes the norm
    with a row factor in its epilogue.  Checked against residual add, norm and products in float32;
    scale_rows() turns the same intermediate into the normalised rows."""
    g = torch.Generator().manual_seed(m * 1000 + h)
    a = (torch.randn(m, k, generator=g)).bfloat16()
    w1 = (torch.randn(h, k, generator=g) / math.sqrt(k)).bfloat16()
    residual = torch.randn(m, h, generator=g) * 3
    gamma = (1 + 0.3 * torch.randn(h, generator=g)).to(w_dtype)
    w2 = (torch.randn(n2, h, generator=g) / math.sqrt(h)).bfloat16()
    bias = None if swiglu else (torch.randn(n2, generator=g)).bfloat16()
    eps = 1e-5

    stream = dev(residual.clone())
    parts = ops.norm_chain_parts(h)
    next_x = torch.empty(m, h, dtype=torch.bfloat16, device="cuda")
    sumsq = torch.full((parts, m), float("nan"), device="cuda")
    ops.gemm_norm_chain(stream, dev(a), dev(w1), accumulate=True, next_x=next_x, next_sumsq=sumsq, next_weight=dev(gamma))
    want_stream = residual + a.float() @ w1.float().T
    torch.testing.assert_close(stream.cpu(), want_stream, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(sumsq.sum(0).cpu(), want_stream.pow(2).sum(1), rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(next_x.cpu().float(), (stream.cpu() * gamma.float()).bfloat16().float(), rtol=0, atol=0)

    normed = want_stream * torch.rsqrt(want_stream.pow(2).mean(1, keepdim=True) + eps) * gamma.float()
    rows = torch.empty(m, h, dtype=torch.bfloat16, device="cuda")
    ops.scale_rows(rows, next_x, sumsq, eps)
    torch.testing.assert_close(rows.cpu().float(), normed, rtol=2e-2, atol=2e-2)

    if swiglu:
        inter = n2 // 2
        gate, up = w2[:inter], w2[inter:]
        stacked = torch.stack((gate.view(inter // 8, 8, h), up.view(inter // 8, 8, h)), 1).reshape(n2, h).contiguous()
        out = torch.empty(m, inter, dtype=torch.bfloat16, device="cuda")
        ops.gemm_norm_chain(out, next_x, dev(stacked), swiglu=True, in_sumsq=sumsq, in_eps=eps)
        want = torch.nn.functional.silu(normed @ gate.float().T) * (normed @ up.float().T)
    else:
        out = torch.empty(m, n2, dtype=torch.bfloat16, device="cuda")
        ops.gemm_norm_chain(out, next_x, dev(w2), dev(bias), in_sumsq=sumsq, in_eps=eps)
        want = normed @ w2.float().T + bias.float()
    close_in_norm(out.float(), want, rel=1.5e-2)


def test_gemm_with_norm_taken_apart_refuses_what_it_cannot_do(ops):
    from llm_runtime_study_amd.errors import KernelError

    a = torch.zeros(17, 64, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(32, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(KernelError, match="at most 16 rows"):
        ops.gemm_norm_chain(torch.zeros(17, 32, device="cuda"), a, w, accumulate=True)
    with pytest.raises(KernelError, match="adds into the residual"):
        ops.gemm_norm_chain(torch.zeros(4, 32, dtype=torch.bfloat16, device="cuda"), a[:4], w,
                            next_x=torch.zeros(4, 32, dtype=torch.bfloat16, device="cuda"),
                            next_sumsq=torch.zeros(2, 4, device="cuda"), next_weight=torch.ones(32, device="cuda"))


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_row_does_not_depend_on_batch(ops, dtype):
    g = torch.Generator().manual_seed(5)
    a = torch.randn(70, 96, generator=g).to(dtype)
    w = torch.randn(200, 96, generator=g).to(dtype)
    full = torch.empty(70, 200, device="cuda")
    ops.gemm(full, dev(a), dev(w))
    one = torch.empty(1, 200, device="cuda")
    ops.gemm(one, dev(a[41:42]), dev(w))
    if dtype == torch.float32:   # one kernel, one order of summation: identical bits
        torch.testing.assert_close(one.cpu(), full.cpu()[41:42], rtol=0, atol=0)
    else:                        # few rows take another kernel than many: equal beyond rounding only
        torch.testing.assert_close(one.cpu(), full.cpu()[41:42], rtol=1e-5, atol=1e-4)
    if dtype == torch.float32:
        # float32 steps of at most 16 rows have a kernel of their own (K a multiple of 64) that adds up in the
        # tiled kernel's order: 3, 8 and 13 rows alone give the bits they have inside a batch of 70
        a64 = torch.randn(70, 192, generator=g)
        w64 = torch.randn(203, 192, generator=g)
        bias = torch.randn(203, generator=g)
        whole = torch.empty(70, 203, device="cuda")
        ops.gemm(whole, dev(a64), dev(w64), dev(bias))
        for first, rows in ((41, 3), (5, 8), (57, 13)):
            few = torch.full((rows, 203), 0.25, device="cuda")
            ops.gemm(few, dev(a64[first:first + rows]), dev(w64), dev(bias))
            torch.testing.assert_close(few.cpu(), whole.cpu()[first:first + rows], rtol=0, atol=0)
            ops.gemm(few, dev(a64[first:first + rows]), dev(w64), dev(bias), accumulate=True)
            torch.testing.assert_close(few.cpu(), 2 * whole.cpu()[first:first + rows], rtol=0, atol=0)
    # strided input and output rows
    wide_in = dev(torch.cat((a, a), 1))
    wide_out = torch.zeros(70, 300, device="cuda")
    ops.gemm(wide_out[:, :200], wide_in[:, 96:], dev(w))
    torch.testing.assert_close(wide_out.cpu()[:, :200], full.cpu(), rtol=0, atol=0)
    assert (wide_out[:, 200:] == 0).all()


def _attention_reference(q, k_all, v_all, positions, lengths_before, nq, nkv, d, scale, window):
    """q [T, nq, d]; k_all/v_all: per request [len, nkv, d]; returns [T, nq*d] float64."""
    outs = []
    for t, (r, p) in enumerate(positions):
        k = k_all[r][: p + 1].double()
        v = v_all[r][: p + 1].double()
        lo = max(0, p - window + 1) if window else 0
        k, v = k[lo:], v[lo:]
        row = []
        for h in range(nq):
            gi = h // (nq // nkv)
            s = (k[:, gi] @ q[t, h].double()) * scale
            row.append(torch.softmax(s, 0) @ v[:, gi])
        outs.append(torch.cat(row))
    return torch.stack(outs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,page,window", [
    (4, 2, 16, 4, 0), (8, 2, 32, 16, 0), (3, 1, 48, 8, 0), (6, 3, 80, 16, 0), (32, 8, 128, 16, 0),
    (4, 4, 256, 64, 0), (8, 2, 32, 16, 7), (4, 2, 64, 16, 33), (16, 1, 96, 32, 0), (12, 4, 192, 16, 21),
    # heads of 128 have a kernel of their own for ragged steps: pages of several runs of 16 keys, kv groups of
    # more heads than a workgroup has waves (several passes) and of fewer, windows
    (8, 1, 128, 32, 0), (6, 2, 128, 64, 40), (16, 1, 128, 16, 21), (2, 2, 128, 48, 0), (5, 1, 128, 16, 70),
])
def test_attention_ragged_batch(ops, dtype, nq, nkv, d, page, window):
    g = torch.Generator().manual_seed(6)
    # request: (cached length before the step, new tokens in the step)
    requests = [(0, 19), (37, 1), (150, 1), (5, 6), (page * 3 - 1, 2), (9, 75)]
    scale = 1 / math.sqrt(d)
    max_blocks = max((a + b + page - 1) // page for a, b in requests)
    n_pages = sum((a + b + page - 1) // page for a, b in requests) + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    kp = torch.zeros(n_pages, nkv, page, d)
    vp = torch.zeros(n_pages, nkv, d, page)
    table = torch.zeros(len(requests), max_blocks, dtype=torch.int32)
    k_all, v_all, q_rows, tok_req, tok_pos, meta = [], [], [], [], [], []
    for r, (before, new) in enumerate(requests):
        total = before + new
        k = torch.randn(total, nkv, d, generator=g).to(dtype)
        v = torch.randn(total, nkv, d, generator=g).to(dtype)
        k_all.append(k.float())
        v_all.append(v.float())
        for b in range((total + page - 1) // page):
            pg = perm.pop()
            table[r, b] = pg
            n = min(page, total - b * page)
            kp[pg, :, :n] = k[b * page: b * page + n].float().transpose(0, 1)
            vp[pg, :, :, :n] = v[b * page: b * page + n].float().permute(1, 2, 0)
        for i in range(new):
            q_rows.append((torch.randn(nq, d, generator=g) * 2).to(dtype))
            tok_req.append(r)
            tok_pos.append(before + i)
            meta.append((r, before + i))
    q = torch.stack(q_rows)
    t = q.shape[0]
    want = _attention_reference(q.float(), k_all, v_all, meta, None, nq, nkv, d, scale, window)
    # q sits in the leading columns of a wider row, as in the fused projection output
    q_wide = torch.zeros(t, nq * d + 2 * nkv * d, dtype=dtype)
    q_wide[:, : nq * d] = q.view(t, nq * d)
    out = torch.empty(t, nq * d, device="cuda", dtype=dtype)
    ops.attention(out, dev(q_wide), dev(kp.to(dtype)), dev(vp.to(dtype)), dev(table),
                  dev(torch.tensor(tok_req, dtype=torch.int32)), dev(torch.tensor(tok_pos, dtype=torch.int32)),
                  nq, scale, window)
    torch.testing.assert_close(out.cpu().double(), want, **tol(dtype, 2e-5, 2e-2))
    if ops.attention_decode_supported(dtype, nq, nkv, d, page):
        # the matrix-core kernel for ragged steps: groups of consecutive tokens of one request, in any order
        assert ops.attention_prefill_group() == 32
        # ... and with the keys of every group divided between several workgroups (more than some groups have tiles)
        for size, splits in ((16, 1), (7, 1), (32, 1), (25, 1), (16, 3), (32, 8), (7, 64)):
            blocks, at = [], 0
            for before, new in requests:
                blocks += [(at + i, min(size, new - i)) for i in range(0, new, size)]
                at += new
            blocks = blocks[::-1]
            fast = torch.empty_like(out)
            part_o = torch.full((out.shape[0], nq * splits * d), float("nan"), device="cuda") if splits > 1 else None
            part_ml = torch.full((out.shape[0], nq * splits * 2), float("nan"), device="cuda") if splits > 1 else None
            ops.attention_prefill(fast, dev(q_wide), dev(kp.to(dtype)), dev(vp.to(dtype)), dev(table),
                                  dev(torch.tensor(tok_req, dtype=torch.int32)), dev(torch.tensor(tok_pos, dtype=torch.int32)),
                                  dev(torch.tensor([b[0] for b in blocks], dtype=torch.int32)),
                                  dev(torch.tensor([b[1] for b in blocks], dtype=torch.int32)), nq, scale, window, size,
                                  splits=splits, part_o=part_o, part_ml=part_ml)
            torch.testing.assert_close(fast.cpu().double(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("nq,nkv,page,window,normed,rotated", [
    (32, 8, 16, 0, True, True), (8, 1, 32, 0, True, True), (6, 2, 64, 40, True, False), (5, 1, 16, 0, False, True), (16, 1, 16, 21, True, True),
])
def test_attention_prefill_prepares_raw_queries(ops, nq, nkv, page, window, normed, rotated):
    """Heads of 128: the kernel for ragged steps given the raw q heads of the q/k/v product (norm and rotation on their
    way into its registers) against attention over queries that were normalised, rotated and rounded beforehand;
    qk_prep(skip_q=True) beside it writes the keys and values as always and leaves the q heads as they were."""
    dtype, d = torch.bfloat16, 128
    g = torch.Generator().manual_seed(61)
    requests = [(0, 19), (37, 1), (150, 1), (5, 6), (page * 3 - 1, 2), (9, 75)]
    scale = 1 / math.sqrt(d)
    max_blocks = max((a + b + page - 1) // page for a, b in requests)
    n_pages = sum((a + b + page - 1) // page for a, b in requests) + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    table = torch.zeros(len(requests), max_blocks, dtype=torch.int32)
    qw = (1 + 0.1 * torch.randn(d, generator=g)).to(dtype) if normed else None
    kw = (1 + 0.1 * torch.randn(d, generator=g)).to(dtype) if normed else None
    rot_half = d // 2 if rotated else 0
    inv = 1.0 / (1e4 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    kp = torch.randn(n_pages, nkv, page, d, generator=g).to(dtype)      # slots not written hold finite junk
    vp = torch.randn(n_pages, nkv, d, page, generator=g).to(dtype)
    rows, slots, tok_req, tok_pos, meta, k_all, v_all = [], [], [], [], [], [], []
    for r, (before, new) in enumerate(requests):
        total = before + new
        for b in range((total + page - 1) // page):
            table[r, b] = perm.pop()
        # what the cache holds of the request before the step, and the raw rows of the step's tokens
        k_old = torch.randn(before, nkv, d, generator=g).to(dtype)
        v_old = torch.randn(before, nkv, d, generator=g).to(dtype)
        for i in range(before):
            pg = int(table[r, i // page])
            kp[pg, :, i % page] = k_old[i]
            vp[pg, :, :, i % page] = v_old[i]
        raw = (torch.randn(new, (nq + 2 * nkv) * d, generator=g) * 2).to(dtype)
        positions = torch.arange(before, total, dtype=torch.int32)
        want_q, want_k, want_v = _qk_prep_reference(raw, nq, nkv, d, qw, kw, 1e-6, positions, inv, rot_half)
        rows.append((raw, want_q.to(dtype).float()))
        k_all.append(torch.cat((k_old.float(), want_k.to(dtype).float())))
        v_all.append(torch.cat((v_old.float(), want_v)))
        for i in range(new):
            slots.append(int(table[r, (before + i) // page]) * page + (before + i) % page)
            tok_req.append(r)
            tok_pos.append(before + i)
            meta.append((r, before + i))
    raw = torch.cat([a for a, _ in rows])
    t = raw.shape[0]
    want = _attention_reference(torch.cat([b for _, b in rows]), k_all, v_all, meta, None, nq, nkv, d, scale, window)
    d_raw, d_kp, d_vp, d_pos = dev(raw), dev(kp), dev(vp), dev(torch.tensor(tok_pos, dtype=torch.int32))
    cos = sin = None
    if rotated:
        cos = torch.empty(t, rot_half, device="cuda")
        sin = torch.empty_like(cos)
        ops.rope_table(cos, sin, d_pos, dev(inv))
    ops.qk_prep(d_raw, nq, nkv, d, None if qw is None else dev(qw), None if kw is None else dev(kw), 1e-6, cos, sin, d_kp, d_vp,
                dev(torch.tensor(slots, dtype=torch.int32)), page, skip_q=True)
    assert torch.equal(d_raw.cpu()[:, :nq * d], raw[:, :nq * d]), "the q heads were to be left alone"
    for i, (r, pos) in enumerate(meta):
        pg = int(table[r, pos // page])
        torch.testing.assert_close(d_kp[pg, :, pos % page].cpu().float(), k_all[r][pos], rtol=2e-2, atol=2e-2)
        assert torch.equal(d_vp[pg, :, :, pos % page].cpu().float(), v_all[r][pos])
    prepare = ops.DecodePrepare(None if qw is None else dev(qw), None, 1e-6, cos, sin, 0)
    for size, splits in ((16, 1), (32, 1), (7, 1), (25, 3), (16, 8)):
        blocks, at = [], 0
        for before, new in requests:
            blocks += [(at + i, min(size, new - i)) for i in range(0, new, size)]
            at += new
        blocks = blocks[::-1]
        out = torch.empty(t, nq * d, device="cuda", dtype=dtype)
        part_o = torch.full((t, nq * splits * d), float("nan"), device="cuda") if splits > 1 else None
        part_ml = torch.full((t, nq * splits * 2), float("nan"), device="cuda") if splits > 1 else None
        ops.attention_prefill(out, d_raw, d_kp, d_vp, dev(table), dev(torch.tensor(tok_req, dtype=torch.int32)), d_pos,
                              dev(torch.tensor([b[0] for b in blocks], dtype=torch.int32)),
                              dev(torch.tensor([b[1] for b in blocks], dtype=torch.int32)), nq, scale, window, size,
                              splits=splits, part_o=part_o, part_ml=part_ml, prepare=prepare)
        torch.testing.assert_close(out.cpu().double(), want, rtol=2e-2, atol=2e-2)
    from llm_runtime_study_amd.errors import KernelError
    with pytest.raises(KernelError):                      # only the queries: no kv heads to write
        ops.attention_prefill(out, d_raw, d_kp, d_vp, dev(table), dev(torch.tensor(tok_req, dtype=torch.int32)), d_pos,
                              dev(torch.tensor([0], dtype=torch.int32)), dev(torch.tensor([1], dtype=torch.int32)), nq, scale, window, 16,
                              prepare=ops.DecodePrepare(None, None, 1e-6, cos, sin, nkv))
    assert not ops.attention_prefill_prepares(64) and ops.attention_prefill_prepares(128)


@pytest.mark.parametrize("nq,nkv,d,page,window,splits", [
    (8, 2, 32, 16, 0, 1), (32, 8, 128, 16, 0, 1), (32, 8, 128, 16, 0, 5), (4, 4, 64, 32, 0, 3), (16, 1, 96, 16, 0, 2),
    (6, 2, 192, 64, 0, 4), (8, 2, 32, 16, 40, 1), (8, 2, 64, 16, 100, 3), (8, 2, 32, 16, 0, 64),
])
def test_attention_decode_kernel(ops, nq, nkv, d, page, window, splits):
    """One query token per request at context lengths around tile and page edges."""
    g = torch.Generator().manual_seed(16)
    lengths = [1, 15, 16, 17, 31, 32, 33, 64, 257, 700]
    scale = 1 / math.sqrt(d)
    blocks = [(n + page - 1) // page for n in lengths]
    n_pages = sum(blocks) + 2
    perm = torch.randperm(n_pages, generator=g).tolist()
    kp = torch.randn(n_pages, nkv, page, d, generator=g)      # slots never written hold finite junk
    vp = torch.randn(n_pages, nkv, d, page, generator=g)
    table = torch.full((len(lengths), max(blocks) + 1), -1, dtype=torch.int32)
    k_all, v_all, meta = [], [], []
    for r, n in enumerate(lengths):
        k = torch.randn(n, nkv, d, generator=g).bfloat16()
        v = torch.randn(n, nkv, d, generator=g).bfloat16()
        k_all.append(k.float())
        v_all.append(v.float())
        for b in range(blocks[r]):
            pg = perm.pop()
            table[r, b] = pg
            m = min(page, n - b * page)
            kp[pg, :, :m] = k[b * page: b * page + m].float().transpose(0, 1)
            vp[pg, :, :, :m] = v[b * page: b * page + m].float().permute(1, 2, 0)
        meta.append((r, n - 1))
    t = len(lengths)
    q = (torch.randn(t, nq, d, generator=g) * 2).bfloat16()
    want = _attention_reference(q.float(), k_all, v_all, meta, None, nq, nkv, d, scale, window)
    q_wide = torch.zeros(t, nq * d + 2 * nkv * d, dtype=torch.bfloat16)
    q_wide[:, : nq * d] = q.view(t, nq * d)
    out = torch.empty(t, nq * d, device="cuda", dtype=torch.bfloat16)
    part_o = torch.empty(t, nq * splits * d, device="cuda")
    part_ml = torch.empty(t, nq * splits * 2, device="cuda")
    assert ops.attention_decode_supported(torch.bfloat16, nq, nkv, d, page)
    # requests sit in another order in the block table than the tokens in the batch
    order = torch.randperm(t, generator=g)
    shuffled = torch.empty_like(table)
    shuffled[order] = table
    results = []
    for form in (0, 1, 2):      # a tile at a time; the next tile on its way, with four and with eight waves
        out.fill_(float("nan"))
        ops.attention_decode(out, dev(q_wide), dev(kp.bfloat16()), dev(vp.bfloat16()), dev(shuffled), dev(order.to(torch.int32)),
                             dev(torch.tensor([n - 1 for n in lengths], dtype=torch.int32)), nq, scale, window, splits, part_o, part_ml,
                             form=form)
        torch.testing.assert_close(out.cpu().double(), want, rtol=2e-2, atol=2e-2)
        results.append(out.cpu().clone())
    assert torch.equal(results[0], results[1])      # the same sums in the same order


@pytest.mark.parametrize("nq,nkv,d,page,window,splits,normed,rotated,shared", [
    (32, 8, 128, 16, 0, 5, True, True, False), (4, 4, 64, 32, 0, 3, True, True, False), (6, 2, 192, 64, 0, 4, False, True, False),
    (8, 2, 32, 16, 0, 2, True, False, False), (16, 1, 96, 16, 40, 1, False, False, False), (8, 2, 64, 16, 100, 3, True, True, True),
    (8, 2, 128, 16, 0, 1, True, True, False),
])
def test_attention_decode_prepares_q_k_v_itself(ops, nq, nkv, d, page, window, splits, normed, rotated, shared):
    """The decode kernel given raw q/k/v rows (it normalises, rotates and writes the new key and
    value itself) against qk_prep() followed by the same kernel: equal outputs and equal pages."""
    g = torch.Generator().manual_seed(23)
    lengths = [1, 15, 16, 17, 31, 32, 33, 64, 257, 700, 48, 49]
    t, scale, eps = len(lengths), 1 / math.sqrt(d), 1e-5
    blocks = [(n + page - 1) // page for n in lengths]
    n_pages = sum(blocks) + 2
    perm = torch.randperm(n_pages, generator=g).tolist()
    kp = torch.randn(n_pages, nkv, page, d, generator=g).bfloat16()   # the new token's slot holds junk
    vp = torch.randn(n_pages, nkv, d, page, generator=g).bfloat16()
    table = torch.full((t, max(blocks) + 1), -1, dtype=torch.int32)
    for r in range(t):
        for b in range(blocks[r]):
            table[r, b] = perm.pop()
    positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32)
    slots = torch.tensor([int(table[r, (n - 1) // page]) * page + (n - 1) % page for r, n in enumerate(lengths)], dtype=torch.int32)
    kv_heads = 0 if shared else nkv
    raw = (torch.randn(t, (nq + 2 * kv_heads) * d, generator=g) * 2).bfloat16()
    qw = (1 + 0.3 * torch.randn(d, generator=g)).bfloat16() if normed else None
    kw = (1 + 0.3 * torch.randn(d, generator=g)).bfloat16() if normed else None
    cos = sin = None
    if rotated:
        angle = torch.rand(t, d // 2, generator=g) * 6.28
        cos, sin = dev(angle.cos()), dev(angle.sin())
    request = dev(torch.arange(t, dtype=torch.int32))

    def run(fused):
        k_dev, v_dev, rows = dev(kp.clone()), dev(vp.clone()), dev(raw.clone())
        out = torch.empty(t, nq * d, device="cuda", dtype=torch.bfloat16)
        part_o = torch.empty(t, nq * splits * d, device="cuda")
        part_ml = torch.empty(t, nq * splits * 2, device="cuda")
        prepare = None
        if fused:
            prepare = ops.DecodePrepare(None if qw is None else dev(qw), None if kw is None else dev(kw), eps, cos, sin, kv_heads)
        else:
            ops.qk_prep(rows, nq, kv_heads, d, None if qw is None else dev(qw), None if kw is None else dev(kw), eps, cos, sin,
                        k_dev, v_dev, dev(slots), page)
        ops.attention_decode(out, rows, k_dev, v_dev, dev(table), request, dev(positions), nq, scale, window, splits,
                             part_o, part_ml, prepare=prepare)
        torch.cuda.synchronize()
        return out.cpu().float(), k_dev.cpu().float(), v_dev.cpu().float()

    assert ops.decode_prepare_supported(d, rotated)
    out_two, k_two, v_two = run(False)
    out_one, k_one, v_one = run(True)
    assert torch.equal(v_one, v_two)
    torch.testing.assert_close(k_one, k_two, rtol=1e-2, atol=1e-6)     # a last bit of bf16 at most
    assert (k_one != kp.float()).any() != shared                        # keys were written, unless they are another layer's
    torch.testing.assert_close(out_one, out_two, rtol=2e-2, atol=2e-2)
    assert (out_one - out_two).norm() <= 4e-3 * out_two.norm()


def test_attention_decode_refuses_to_rotate_odd_chunk_counts(ops):
    from llm_runtime_study_amd.errors import KernelError

    assert not ops.decode_prepare_supported(96, True) and ops.decode_prepare_supported(96, False)
    kp = torch.zeros(2, 1, 16, 96, dtype=torch.bfloat16, device="cuda")
    vp = torch.zeros(2, 1, 96, 16, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(KernelError, match="cannot rotate"):
        ops.attention_decode(torch.zeros(1, 96, dtype=torch.bfloat16, device="cuda"), torch.zeros(1, 3 * 96, dtype=torch.bfloat16, device="cuda"),
                             kp, vp, torch.zeros(1, 2, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda"),
                             torch.zeros(1, dtype=torch.int32, device="cuda"), 1, 0.1,
                             prepare=ops.DecodePrepare(None, None, 1e-6, torch.zeros(1, 48, device="cuda"), torch.zeros(1, 48, device="cuda"), 1))


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_a_far_key(ops, dtype):
    """One key among 700 is made to dominate: the output must be its value, wherever it lies."""
    nq, nkv, d, page = 2, 1, 32, 16
    g = torch.Generator().manual_seed(7)
    length = 700
    for far in (0, 15, 16, 127, 128, 511, 698, 699):
        k = torch.randn(length, nkv, d, generator=g) * 0.1
        v = torch.randn(length, nkv, d, generator=g)
        q = torch.randn(1, nq, d, generator=g)
        q = q / q.norm(dim=-1, keepdim=True)
        k[far, 0] = q[0, 0] * 60  # score 60/sqrt(32)*... dominates head 0
        n_pages = (length + page - 1) // page
        kp = torch.zeros(n_pages, nkv, page, d)
        vp = torch.zeros(n_pages, nkv, d, page)
        order = torch.randperm(n_pages, generator=g)
        table = order.to(torch.int32).view(1, -1)
        for b in range(n_pages):
            n = min(page, length - b * page)
            kp[order[b], :, :n] = k[b * page: b * page + n].transpose(0, 1)
            vp[order[b], :, :, :n] = v[b * page: b * page + n].permute(1, 2, 0)
        out = torch.empty(1, nq * d, device="cuda", dtype=dtype)
        ops.attention(out, dev(q.view(1, -1).to(dtype)), dev(kp.to(dtype)), dev(vp.to(dtype)), dev(table),
                      dev(torch.zeros(1, dtype=torch.int32)), dev(torch.tensor([length - 1], dtype=torch.int32)), nq, 1.0, 0)
        torch.testing.assert_close(out.cpu().float()[0, :d], v[far, 0].to(dtype).float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("window,planted", [(0, 0), (0, 17), (0, 527), (100, 600), (100, 599), (100, 595), (100, 689), (33, 660)])
def test_one_key_stands_out_in_every_attention_kernel(ops, window, planted):
    """Ten new tokens after 690 cached ones, every query pointing at one planted key whose score dwarfs the
    rest.  Without a window every query must return that key's value, wherever it lies (first tile, a page
    edge, deep in the cache); with a window the key counts for exactly the queries whose window still holds
    it (595 with a window of 100: positions 690..694 yes, 695..699 no; 599: only 690..698) and a kernel
    that is one off at the window's edge returns a different row.  All kernels: the general one, the
    matrix-core decode kernel (last token; whole and split over keys) and the ragged prefill kernel."""
    run_one_key_stands_out(ops, window, planted, 64, 16)
    run_one_key_stands_out(ops, window, planted, 128, 16)      # heads of 128: the ragged kernel is another one
    run_one_key_stands_out(ops, window, planted, 128, 32)


@pytest.mark.parametrize("window,planted", [(0, 0), (0, 32767), (0, 32768), (0, 39001), (100, 39950), (100, 39895)])
def test_one_key_stands_out_far_back_in_a_long_context(ops, window, planted):
    """The same ten tokens after 39,990 cached ones (2,500 pages of 16, or 625 of 64): block tables, key numbers and
    byte offsets of a size the short tests never reach, in every attention kernel and with the keys divided."""
    run_one_key_stands_out(ops, window, planted, 128, 16, before=39990)
    run_one_key_stands_out(ops, window, planted, 64, 64, before=39990)


def run_one_key_stands_out(ops, window, planted, d, page, before=690):
    nq, nkv, new = 4, 2, 10
    length = before + new
    g = torch.Generator().manual_seed(70 + planted)
    k = (torch.randn(length, nkv, d, generator=g) * 0.1).bfloat16()
    v = torch.randn(length, nkv, d, generator=g).bfloat16()
    direction = torch.randn(d, generator=g)
    direction = direction / direction.norm()
    k[planted] = (direction * 40).bfloat16()
    q = (direction * 2).bfloat16().expand(new, nq, d).contiguous()      # score 80 * scale at the planted key
    scale = 1.0
    n_pages = (length + page - 1) // page
    order = torch.randperm(n_pages + 2, generator=g)[:n_pages]
    kp = torch.randn(n_pages + 2, nkv, page, d, generator=g)
    vp = torch.randn(n_pages + 2, nkv, d, page, generator=g)
    for b in range(n_pages):
        n = min(page, length - b * page)
        kp[order[b], :, :n] = k[b * page: b * page + n].float().transpose(0, 1)
        vp[order[b], :, :, :n] = v[b * page: b * page + n].float().permute(1, 2, 0)
    table = order.to(torch.int32).view(1, -1)
    meta = [(0, before + i) for i in range(new)]
    want = _attention_reference(q.float(), [k.float()], [v.float()], meta, None, nq, nkv, d, scale, window)
    for i, (_, pos) in enumerate(meta):     # the scenario is what the docstring says
        seen = planted <= pos and (window == 0 or planted > pos - window)
        close = torch.allclose(want[i, :d], v[planted, 0].double(), atol=1e-2)
        assert close == seen, (pos, seen)
    q_wide = torch.zeros(new, (nq + 2 * nkv) * d, dtype=torch.bfloat16)
    q_wide[:, : nq * d] = q.view(new, nq * d)
    request = dev(torch.zeros(new, dtype=torch.int32))
    positions = dev(torch.tensor([pos for _, pos in meta], dtype=torch.int32))
    pages = (dev(kp.bfloat16()), dev(vp.bfloat16()))
    out = torch.full((new, nq * d), float("nan"), device="cuda", dtype=torch.bfloat16)
    ops.attention(out, dev(q_wide), *pages, dev(table), request, positions, nq, scale, window)
    torch.testing.assert_close(out.cpu().double(), want, rtol=2e-2, atol=2e-2)
    for splits in (1, 4, 11):
        last = torch.full((1, nq * d), float("nan"), device="cuda", dtype=torch.bfloat16)
        part_o = torch.full((1, nq * splits * d), float("nan"), device="cuda")
        part_ml = torch.full((1, nq * splits * 2), float("nan"), device="cuda")
        for form in (0, 1, 2):
            ops.attention_decode(last, dev(q_wide[-1:]), *pages, dev(table), request[:1], positions[-1:], nq, scale, window,
                                 splits, part_o, part_ml, form=form)
            torch.testing.assert_close(last.cpu().double(), want[-1:], rtol=2e-2, atol=2e-2)
    for size, splits in ((16, 1), (32, 1), (4, 1), (16, 5), (32, 16)):
        groups = [(i, min(size, new - i)) for i in range(0, new, size)]
        fast = torch.full((new, nq * d), float("nan"), device="cuda", dtype=torch.bfloat16)
        part_o = torch.full((new, nq * splits * d), float("nan"), device="cuda") if splits > 1 else None
        part_ml = torch.full((new, nq * splits * 2), float("nan"), device="cuda") if splits > 1 else None
        ops.attention_prefill(fast, dev(q_wide), *pages, dev(table), request, positions,
                              dev(torch.tensor([b[0] for b in groups], dtype=torch.int32)),
                              dev(torch.tensor([b[1] for b in groups], dtype=torch.int32)), nq, scale, window, size,
                              splits=splits, part_o=part_o, part_ml=part_ml)
        torch.testing.assert_close(fast.cpu().double(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("rows,vocab", [(1, 256), (5, 331), (3, 151936), (5, 20000)])
def test_choose_tokens_greedy(ops, rows, vocab):
    g = torch.Generator().manual_seed(8)
    logits = torch.randn(rows, vocab, generator=g)
    logits[0, vocab - 1] = 50.0
    if rows > 1:
        logits[1, 5] = logits[1, 77] = 40.0  # tie: the lowest index wins
    if rows > 2:
        logits[2, 100] = logits[2, vocab - 7] = 45.0  # a tie between far-apart slices of the vocabulary
    out = torch.empty(rows, dtype=torch.int32, device="cuda")
    ops.choose_tokens(out, dev(logits))
    want = [vocab - 1, 5, 100] + [int(torch.argmax(logits[i])) for i in range(3, rows)]
    assert out.cpu().tolist() == want[:rows]


def test_choose_tokens_two_pass_equals_one_pass(ops):
    """Large vocabularies take the two-pass kernels: same choice as the one-pass kernel, sampled rows included."""
    rows, vocab = 6, 151936
    g = torch.Generator().manual_seed(18)
    logits = dev(torch.randn(rows, vocab, generator=g) * 2)
    temps = dev(torch.tensor([0.0, 0.7, 1.0, 1.5, 0.0, 0.3]))
    seeds = dev(torch.tensor([1, 2, 3, 4, 5, 6], dtype=torch.int64))
    counters = dev(torch.tensor([0, 9, 2, 7, 1, 4], dtype=torch.int32))
    two = torch.empty(rows, dtype=torch.int32, device="cuda")
    ops.choose_tokens(two, logits, temps, seeds, counters)
    one = torch.empty(rows, dtype=torch.int32, device="cuda")
    code = ops.library().lrs_choose_tokens(one.data_ptr(), logits.data_ptr(), vocab, rows, vocab, temps.data_ptr(), seeds.data_ptr(),
                                           counters.data_ptr(), 0, torch.cuda.current_stream().cuda_stream)
    assert code == 0 and one.cpu().tolist() == two.cpu().tolist()
    assert two.cpu()[0] == logits[0].argmax().cpu() and two.cpu()[1] != logits[1].argmax().cpu()


def test_choose_tokens_temperature_statistics(ops):
    vocab, draws = 11, 20000
    probs = torch.tensor([0.3, 0.2, 0.15, 0.1, 0.08, 0.07, 0.05, 0.03, 0.01, 0.01, 0.0])
    temperature = 0.7
    logits = (torch.log(probs) * temperature).repeat(draws, 1)  # softmax(logits / T) = probs
    out = torch.empty(draws, dtype=torch.int32, device="cuda")
    temps = torch.full((draws,), temperature, device="cuda")
    seeds = torch.full((draws,), 1234, dtype=torch.int64, device="cuda")
    counters = torch.arange(draws, dtype=torch.int32, device="cuda")
    ops.choose_tokens(out, dev(logits), temps, seeds, counters, filtered=True)   # -inf as a filter leaves it
    freq = torch.bincount(out.cpu().long(), minlength=vocab).float() / draws
    assert freq[-1] == 0  # a -inf logit is never drawn
    assert (freq - probs).abs().max() < 0.012
    # reproducible, and a row's draw does not depend on its neighbours
    again = torch.empty(7, dtype=torch.int32, device="cuda")
    ops.choose_tokens(again, dev(logits[:7]), temps[:7], seeds[:7], counters[100:107].contiguous(), filtered=True)
    assert again.cpu().tolist() == out.cpu()[100:107].tolist()
    other = torch.empty(draws, dtype=torch.int32, device="cuda")
    ops.choose_tokens(other, dev(logits), temps, seeds + 1, counters, filtered=True)
    assert (other != out).float().mean() > 0.3


@pytest.mark.parametrize("vocab", [1000, 151936], ids=["one-pass", "two-pass"])
def test_rows_that_are_not_finite_are_refused(ops, vocab):
    """The reference refuses logits that hold a value that is not finite (mini_llm/sampling.py:104-113): here such a
    row's token comes out as -1 beside healthy rows, greedy or drawn, filtered or not, and the sampler raises."""
    from llm_runtime_study_amd.errors import SamplingError
    from llm_runtime_study_amd.sampling import Sampler, SamplingConfig, SamplingRow

    g = torch.Generator().manual_seed(21)
    base = torch.randn(6, vocab, generator=g)
    base[1, vocab - 3] = float("nan")
    base[3, 17] = float("inf")
    base[4, vocab // 2] = float("-inf")
    base[5, :] = float("-inf")                       # nothing to choose from
    out = torch.empty(6, dtype=torch.int32, device="cuda")
    ops.choose_tokens(out, dev(base))
    assert out.cpu().tolist() == [int(base[0].argmax()), -1, int(base[2].argmax()), -1, -1, -1]
    # drawn rows without a filter: the same rows are refused
    temps = torch.full((6,), 0.8, device="cuda")
    seeds = torch.arange(6, dtype=torch.int64, device="cuda")
    counters = torch.zeros(6, dtype=torch.int32, device="cuda")
    ops.choose_tokens(out, dev(base), temps, seeds, counters)
    got = out.cpu().tolist()
    assert [t < 0 for t in got] == [False, True, False, True, True, True] and all(t < vocab for t in got)
    # after filter_logits() a -inf is what a filter leaves, but the rows that came with one are still refused:
    # the filter marks them; a greedy row among them (temperature 0) is never filtered and is looked at as it came
    work = dev(base.clone())
    temps = torch.tensor([0.8, 0.8, 0.0, 0.8, 0.8, 0.8], device="cuda")
    ks = torch.tensor([5, 5, 0, 0, 5, 5], dtype=torch.int32, device="cuda")
    ps = torch.tensor([1.0, 1.0, 1.0, 0.9, 1.0, 0.5], device="cuda")
    ops.filter_logits(work, temps, ks, ps)
    ops.choose_tokens(out, work, temps, seeds, counters, filtered=True)
    got = out.cpu().tolist()
    assert [t < 0 for t in got] == [False, True, False, True, True, True]
    assert got[2] == int(base[2].argmax()) and got[0] in base[0].topk(5).indices.tolist()
    assert torch.isfinite(work[0]).sum().item() == 5 and torch.isfinite(work[2]).all()

    sampler = Sampler("cuda")
    for config in (SamplingConfig(), SamplingConfig(temperature=0.8, seed=1), SamplingConfig(temperature=0.8, top_k=7, seed=1),
                   SamplingConfig(temperature=0.8, top_p=0.9, seed=1)):
        rows = [SamplingRow(config, 1, 0)] * 2
        healthy = sampler.choose(dev(base[[0, 2]].clone()), rows)
        assert all(0 <= t < vocab for t in healthy)
        for bad in (1, 3, 4):
            with pytest.raises(SamplingError, match="only finite values"):
                sampler.choose(dev(base[[0, bad]].clone()), rows)


def test_filter_logits_matches_sort_based_rule(ops):
    from tests.plain.model import filter_logits as plain_filter

    g = torch.Generator().manual_seed(9)
    cases = [(0.8, 5, 1.0), (1.3, None, 0.7), (0.5, 40, 0.9), (1.0, 1, 0.5), (2.0, None, 0.05), (1.0, 331, 1.0)]
    logits = torch.randn(len(cases), 331, generator=g) * 3
    logits[1, :4] = torch.log(torch.tensor([0.60, 0.25, 0.10, 0.05])) + 30  # reference vector: p=.70 keeps two
    work = dev(logits.clone())
    temps = dev(torch.tensor([c[0] for c in cases]))
    ks = dev(torch.tensor([c[1] or 0 for c in cases], dtype=torch.int32))
    ps = dev(torch.tensor([c[2] for c in cases]))
    ops.filter_logits(work, temps, ks, ps)
    got = work.cpu()
    for i, (temp, k, p) in enumerate(cases):
        want = plain_filter(logits[i], temp, k, p)
        assert torch.equal(torch.isfinite(got[i]), torch.isfinite(want)), f"case {i}"
        kept = torch.isfinite(want)
        torch.testing.assert_close(got[i][kept], logits[i][kept], rtol=0, atol=0)
    assert torch.isfinite(got[1]).sum() == 2


def test_filter_logits_compares_the_scaled_values(ops):
    """The thresholds are values of logits / temperature (mini_llm/sampling.py:53-64), not of the logits: two logits
    one step of float32 apart whose quotients round to one float32 are a tie.  At the k-th place the reference's
    topk keeps one of the two, whichever; here both stay, and nothing else differs."""
    from tests.plain.model import filter_logits as plain_filter

    temp, k, vocab = 0.7, 6, 400
    low = torch.tensor(1.5)
    while True:                                       # neighbours whose quotients by the temperature are one float32
        high = torch.nextafter(low, torch.tensor(2.0))
        if low / temp == high / temp:
            break
        low = high
    assert low != high
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(2, vocab, generator=g).clamp(max=1.2)
    logits[:, 10:15] = torch.tensor([3.0, 2.9, 2.8, 2.7, 2.6])      # five above the pair
    logits[:, 200], logits[:, 300] = high, low                      # the k-th and the one after it
    work = dev(logits.clone())
    temps = dev(torch.tensor([temp, temp]))
    ops.filter_logits(work, temps, dev(torch.tensor([k, 0], dtype=torch.int32)), dev(torch.tensor([1.0, 0.999])))
    kept = torch.isfinite(work.cpu())
    assert kept[0].sum() == k + 1 and kept[0, 200] and kept[0, 300]
    want = torch.isfinite(plain_filter(logits[0], temp, k, 1.0))
    assert want.sum() == k and want[200] != want[300]
    others = torch.ones(vocab, dtype=torch.bool)
    others[[200, 300]] = False
    assert torch.equal(kept[0][others], want[others])
    # the mass rule likewise: the pair is kept or dropped together
    assert kept[1, 200] == kept[1, 300]


@pytest.mark.parametrize("vocab", [151936, 50257, 4099])
def test_filter_logits_of_a_large_vocabulary_matches_the_sort_based_rule(ops, vocab):
    """The selection by digits of the bit pattern, where it has something to select from: a vocabulary of the
    real size, rows whose values crowd into one or two of its first bins (all between 16 and 20; all negative
    and small), rows with the usual spread, a k beyond the first bin, a share that the largest value holds alone."""
    from tests.plain.model import filter_logits as plain_filter

    g = torch.Generator().manual_seed(vocab)
    cases = [(0.8, 50, 1.0), (1.0, None, 0.9), (0.7, 50, 0.9), (1.0, 1000, 0.95), (1.5, 7, 0.3), (1.0, None, 0.999),
             (1.0, 20, 0.9), (1.0, None, 0.5), (0.9, 3000, 1.0), (1.0, None, 0.2)]
    logits = torch.randn(len(cases), vocab, generator=g) * 3
    logits[6] = 16 + 4 * torch.rand(vocab, generator=g)          # one bin of the first digit holds them all
    logits[7] = -1e-3 * torch.rand(vocab, generator=g) - 1e-4    # tiny negatives, close together
    logits[9, 17] = 40.0                                         # one token has nearly all the mass
    work = dev(logits.clone())
    temps = dev(torch.tensor([c[0] for c in cases]))
    ks = dev(torch.tensor([c[1] or 0 for c in cases], dtype=torch.int32))
    ps = dev(torch.tensor([c[2] for c in cases]))
    ops.filter_logits(work, temps, ks, ps)
    got = work.cpu()
    def rule_in_float64(row, temp, k, p):
        # tests/plain/model.py:filter_logits with the masses added up in float64 (in float32 the running sum of
        # 150,000 terms is itself uncertain by more than the tokens at the edge of a share of 0.999 weigh)
        z = (row.float() / temp).double()
        if k is not None and k < z.numel():
            top, idx = torch.topk(z, k)
            z = torch.full_like(z, -torch.inf).scatter(0, idx, top)
        if p < 1.0:
            ordered, idx = torch.sort(z, descending=True)
            share = torch.softmax(ordered, -1)
            before = torch.cumsum(share, -1) - share
            z = torch.empty_like(z).scatter(0, idx, ordered.masked_fill(before >= p, -torch.inf))
        return z

    for i, (temp, k, p) in enumerate(cases):
        if vocab == 4099:
            assert torch.equal(torch.isfinite(plain_filter(logits[i], temp, k, p)), torch.isfinite(rule_in_float64(logits[i], temp, k, p)))
        kept, wanted = torch.isfinite(got[i]), torch.isfinite(rule_in_float64(logits[i], temp, k, p))
        # a token exactly at the edge may fall either way (the kernel's exponentials are float32); far down the tail
        # (a share of 0.999) a few more, but never a mass that matters
        share = torch.softmax(logits[i].double() / temp, -1)
        assert share[kept != wanted].sum() < 2e-7, f"case {i}: {kept.sum()} kept, {wanted.sum()} wanted"
        if p < 0.99:
            assert (kept != wanted).sum() <= 1, f"case {i}: {kept.sum()} kept, {wanted.sum()} wanted"
        both = kept & wanted
        torch.testing.assert_close(got[i][both], logits[i][both], rtol=0, atol=0)
        if k is not None and p == 1.0:
            assert torch.equal(kept, wanted) and kept.sum() == k
    assert torch.isfinite(got[9]).sum() == 1


@pytest.mark.gpu
def test_the_probes_of_lds_and_matrix_rates_run_and_refuse_what_they_cannot_do(ops):
    """`microbench lds`, `microbench mfma` and `microbench lines` are measurements, not products: here only that
    they launch, finish and refuse parameters outside what their kernels hold."""
    from llm_runtime_study_amd.errors import KernelError

    ints = torch.zeros(256, dtype=torch.int32, device="cuda")
    floats = torch.zeros(256, dtype=torch.float32, device="cuda")
    ops.probe_lds(ints, 8, 4, 96)
    ops.probe_mfma(floats, 8, 4, 2, True)
    ops.probe_mfma(floats, 8, 4, 0, False)
    data = torch.zeros(3 * 8192 // 4, dtype=torch.int32, device="cuda")
    for pattern in range(3):
        ops.probe_lines(data, ints, 3, 256, 8192, pattern)
    ops.probe_lines(data, ints, 1, 1024, 3 * 8192, 1)
    torch.cuda.synchronize()
    for blocks, threads, each, pattern in ((4, 256, 8192, 0), (3, 96, 8192, 0), (3, 256, 6000, 1), (3, 256, 8192, 3)):   # beyond the data; no whole waves; no whole turns
        with pytest.raises(KernelError):
            ops.probe_lines(data, ints, blocks, threads, each, pattern)
    for bad in (8, 100, 1024):
        with pytest.raises(KernelError):
            ops.probe_lds(ints, 8, 4, bad)
    with pytest.raises(KernelError):
        ops.probe_mfma(floats, 8, 4, 5, False)
