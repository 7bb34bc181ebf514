"""Each HIP kernel alone against its plain reference (the test stand-in, written with
elementary tensor operations), at sizes other than the engine's: head sizes 16 to 256,
one to eight query heads per key/value head, widths and vocabularies that are no power
of two. Inputs are built so that a fault shows: a far key that must win, the edge of a
window, a block boundary of the cache."""
import math
from types import SimpleNamespace

import pytest
import torch

import cache_order
from ops_emulation import EmulatedOps
import plain_llama as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# elementwise kernels round once: half a unit in the last place of the output type
ULP = {"float32": 2e-6, "bfloat16": 4e-3}


@pytest.fixture(scope="module")
def ops():
    from xeno_rt_amd.ops import load_ops
    return load_ops()


REF = EmulatedOps()


def rand(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def packed_or_not(ops, w, packed, kind="tiles", **details):
    """w as the products take it: as it is, or in the tiled layout (bfloat16, k a multiple of 32)."""
    if not packed:
        return w
    if w.dtype != torch.bfloat16 or w.shape[1] % 32 != 0:
        pytest.skip("only bfloat16 matrices whose k is a multiple of 32 are packed")
    return ops.pack(w, kind, **details)


def rel(got, want):
    return float((got.double() - want.double()).abs().max()) / max(1e-30, float(want.double().abs().max()))


# ---- embedding, add, rmsnorm -----------------------------------------------------------

@pytest.mark.parametrize("hidden", [200, 201, 4096])          # rows of 16-byte pieces, rows that are not, rows longer than a workgroup's step
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed_and_add(ops, dtype, hidden):
    table = rand(777, hidden, dtype=DT[dtype])
    ids = torch.tensor([0, 776, 5, 5, 123], dtype=torch.int32, device=DEV)
    out = torch.empty(5, hidden, device=DEV)
    ops.embed(table, ids, out)
    assert torch.equal(out, table[ids.long()].float())
    delta = rand(5, hidden, dtype=DT[dtype], seed=2)
    want = out + delta.float()
    ops.add(out, delta)
    assert torch.equal(out, want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hidden", [1, 96, 1000, 5120])
def test_rmsnorm(ops, dtype, hidden):
    x = rand(7, hidden, seed=hidden, scale=3.0)
    for weight in (rand(hidden, seed=1) + 1.0, (rand(hidden, seed=1) + 1.0).to(torch.bfloat16)):
        out = torch.empty(7, hidden, dtype=DT[dtype], device=DEV)
        ops.rmsnorm(x, weight, 1e-3, out)
        want = P.rmsnorm(x.double().cpu(), weight.double().cpu(), 1e-3)
        assert rel(out.cpu(), want) < ULP[dtype]
        rows = torch.tensor([6, 0, 6], dtype=torch.int32, device=DEV)
        picked = torch.empty(3, hidden, dtype=DT[dtype], device=DEV)
        ops.rmsnorm(x, weight, 1e-3, picked, rows=rows)
        assert torch.equal(picked, out[rows.long()])          # a row's result does not depend on the batch


def test_rmsnorm_reference_vector(ops):
    # tests/kernels_test.rs:75-91 of the reference
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]], device=DEV)
    w = torch.tensor([1.0, 1.5, 2.0, 2.5], device=DEV)
    out = torch.empty(1, 4, device=DEV)
    ops.rmsnorm(x, w, 1e-5, out)
    inv = 1.0 / math.sqrt(7.5 + 1e-5)
    assert rel(out.cpu(), torch.tensor([[inv, 3 * inv, 6 * inv, 10 * inv]])) < 1e-6


# ---- matrix products -----------------------------------------------------------------------

SHAPES = [(1, 64, 64), (3, 200, 96), (8, 1000, 176), (17, 96, 192), (64, 333, 520), (130, 257, 72),
          (300, 520, 1032), (1, 3, 5), (5, 7, 13), (33, 4100, 264), (64, 40, 4096), (65, 40, 4096),
          (2048, 6144, 128), (2000, 6200, 136), (70, 300, 64), (300, 520, 1024), (2100, 6100, 320),
          (2100, 8300, 128), (40, 4100, 1024), (64, 333, 640), (33, 130, 128), (17, 700, 192),
          (600, 520, 8192), (520, 1030, 8320),         # many rows, few columns, a very long k (large tiles that split k)
          (12, 8200, 288), (9, 8208, 1056), (16, 16400, 4096), (16, 8192, 4128),   # 9 to 16 rows, many rows of w, k up to 4096: x stays in registers (the last: k too long for that)
          # 65 to 256 rows, too few columns to fill the chip: tiles of 128 x 64 that split k in long parts (the last two: a long k keeps tiles of 128 x 128, in three stages)
          (72, 4096, 4096), (130, 1000, 2048), (256, 4104, 1024), (200, 700, 4160), (100, 2048, 8192), (250, 1030, 14336)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "bfloat16 packed"])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_linear(ops, dtype, m, n, k):
    dtype, packed = dtype.split()[0], dtype.endswith("packed")
    a = rand(m, k, dtype=DT[dtype], seed=m)
    w = rand(n, k, dtype=DT[dtype], seed=n, scale=0.1)
    want = a.double().cpu() @ w.double().cpu().t()
    w = packed_or_not(ops, w, packed)
    out32 = torch.empty(m, n, device=DEV)
    ops.linear(a, w, out32)
    assert rel(out32.cpu(), want) < 1e-5                        # float32 accumulation in both paths
    out = torch.empty(m, n, dtype=DT[dtype], device=DEV)
    ops.linear(a, w, out)
    assert rel(out.cpu(), want) < ULP[dtype] * 2
    base = rand(m, n, seed=5)
    acc = base.clone()
    ops.linear(a, w, acc, accumulate=True)
    assert rel(acc.cpu(), base.double().cpu() + want) < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "bfloat16 packed"])
@pytest.mark.parametrize("m,n,k", [(1, 176, 64), (9, 100, 96), (64, 520, 200), (200, 1000, 72), (48, 2000, 520),
                                   (3, 8, 32), (16, 24, 160), (30, 1000, 96), (64, 4104, 224), (8, 14336, 4096),
                                   (2048, 3100, 64), (300, 130, 1032), (2048, 3072, 128), (2000, 3000, 192), (2048, 4224, 64),
                                   (64, 520, 256), (50, 1000, 1024), (200, 1000, 512),
                                   # 17 to 64 rows and tiles enough without a split along k
                                   (40, 14336, 256), (64, 9002, 128), (33, 20000, 192),
                                   # 9 to 16 rows and many pairs: x stays in the registers of a workgroup that walks the rows of w
                                   (13, 4104, 96), (16, 14336, 4096), (9, 8192, 2080),
                                   # 65 to 128 rows and about a round of tiles of 128 x 128: no split, three stages
                                   (72, 14336, 1024), (128, 13000, 512), (100, 15000, 192)])
def test_linear_glu(ops, dtype, m, n, k):
    dtype, packed = dtype.split()[0], dtype.endswith("packed")
    if packed and n % 8 != 0:
        pytest.skip("gate and up rows are paired in groups of 8")
    a = rand(m, k, dtype=DT[dtype], seed=1)
    w = rand(2 * n, k, dtype=DT[dtype], seed=2, scale=0.3)
    both = a.double().cpu() @ w.double().cpu().t()
    want = P.swiglu(both[:, :n], both[:, n:])
    w = packed_or_not(ops, w, packed, "gated", gated_n=n)
    out = torch.empty(m, n, dtype=DT[dtype], device=DEV)
    ops.linear_glu(a, w, out)
    assert rel(out.cpu(), want) < ULP[dtype] * 2


def test_linear_of_more_elements_than_32_bit_offsets_reach(ops):
    """x with 2^31 elements and more (a step of many long prompts times a wide feed-forward) goes through the
    matrix-core kernels in runs of rows: rows at the runs' edges are right, and the same as in a product of their own."""
    k, n = 16384, 96
    run = (2 ** 31 - 1) // k // 256 * 256
    m = 2 ** 31 // k + 300                                      # two runs, the second short
    assert run < m and m * k > 2 ** 31
    generator = torch.Generator(device=DEV).manual_seed(3)
    a = torch.empty(m, k, dtype=torch.bfloat16, device=DEV)
    for begin in range(0, m, 16384):                             # filled piecewise: no float32 copy of 8 GB
        a[begin:begin + 16384] = torch.randn(min(16384, m - begin), k, generator=generator, device=DEV) * 0.5
    w = rand(2 * n, k, dtype=torch.bfloat16, seed=4, scale=0.05)
    rows = [0, 1000, run - 1, run, run + 1, m - 1]
    out = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    ops.linear_glu(a, w, out)
    acc = torch.zeros(m, 2 * n, device=DEV)
    ops.linear(a, w, acc, accumulate=True)
    torch.cuda.synchronize()
    picked = a[rows].contiguous()
    both = picked.double().cpu() @ w.double().cpu().t()
    assert rel(acc[rows].cpu(), both) < 1e-5
    assert rel(out[rows].cpu(), P.swiglu(both[:, :n], both[:, n:])) < ULP["bfloat16"] * 2
    across = torch.zeros(512, 2 * n, device=DEV)                 # the rows on both sides of the edge, as one product
    ops.linear(a[run - 256:run + 256].contiguous(), w, across, accumulate=True)
    assert rel(across.cpu(), acc[run - 256:run + 256].cpu().double()) < 1e-5    # (split along k: another order of the sum)


def test_linear_rows_do_not_depend_on_the_batch(ops):
    a = rand(70, 200, seed=3)
    w = rand(130, 200, seed=4)
    whole = torch.empty(70, 130, device=DEV)
    ops.linear(a, w, whole)
    for row in (0, 63, 64, 69):
        one = torch.empty(1, 130, device=DEV)
        ops.linear(a[row:row + 1].contiguous(), w, one)
        assert torch.equal(one[0], whole[row])                  # same bits: same order of the sum


@pytest.mark.parametrize("m,hidden,k,n", [(1, 4096, 512, 1024), (8, 4096, 14336, 6144), (16, 200, 96, 72),
                                          (5, 1000, 136, 333), (13, 8200, 64, 48), (13, 4096, 64, 4104), (16, 1056, 96, 8200),
                                          (17, 4096, 512, 1024), (40, 1024, 256, 333), (64, 4096, 14336, 6144), (33, 512, 128, 20000)])
@pytest.mark.parametrize("packed", [False, True])
def test_rmsnorm_done_by_the_products_around_it(ops, m, hidden, k, n, packed):
    # x += a w^T; y = rmsnorm(x) * gain; z = y v^T (and the gated pair), the norm without a kernel of its own:
    # up to 16 rows in the kernel that streams w, 17 to 64 rows in the tiles split along k and their second kernel
    a = rand(m, k, dtype=torch.bfloat16, seed=1)
    w = rand(hidden, k, dtype=torch.bfloat16, seed=2, scale=0.2)
    x = rand(m, hidden, seed=3, scale=2.0)
    x[m // 2] *= 50.0                                            # rows of different size: each needs its own rms
    eps = 1e-3
    # a row whose mean square is about eps, and a row of zeros: only an eps that is added once, inside the root,
    # gives the first its scale (doubled, it would be a fifth off) and the second zeros instead of NaN
    small, zero = (0, m - 1) if m >= 3 else (None, None)
    if small is not None:
        a[small], a[zero] = 0.0, 0.0
        x[small], x[zero] = rand(hidden, seed=7, scale=0.03), 0.0
    gain = (rand(hidden, seed=4) + 1.0).to(torch.bfloat16)
    v = rand(2 * n, hidden, dtype=torch.bfloat16, seed=5, scale=0.1)
    fresh = x.double().cpu() + a.double().cpu() @ w.double().cpu().t()
    normed = P.rmsnorm(fresh, gain.double().cpu(), eps)
    plain_v = v
    if packed and (hidden % 32 != 0 or n % 8 != 0):
        pytest.skip("sizes that are not packed")
    w = packed_or_not(ops, w, packed)
    v_glu = packed_or_not(ops, v, packed, "gated", gated_n=n)
    v = packed_or_not(ops, v, packed)

    scaled = ops.linear(a, w, x, accumulate=True, then_norm=(gain, eps))
    if packed and hidden % 16 != 0 and m <= 16:
        assert scaled is None                                   # a packed w writes sums of squares per tile of 16 columns
        return
    assert scaled is not None and scaled.shape == (m, hidden)
    assert rel(x.cpu(), fresh) < 1e-5
    tiles = scaled.squares.shape[0]                 # the product cuts its columns into tiles of 16 or fewer, all alike
    width = -(-hidden // tiles)
    assert 8 <= width <= 16 and tiles == -(-hidden // width)
    padded = torch.zeros(m, tiles * width, dtype=torch.float64)
    padded[:, :hidden] = x.double().cpu() ** 2
    assert rel(scaled.squares[:, :m].t().cpu(), padded.reshape(m, tiles, width).sum(-1)) < 1e-6
    assert rel(scaled.values.cpu(), x.double().cpu() * gain.double().cpu()) < ULP["bfloat16"]

    want = normed @ plain_v.double().cpu().t()
    for out_dtype in (torch.float32, torch.bfloat16):
        out = torch.empty(m, 2 * n, dtype=out_dtype, device=DEV)
        ops.linear(scaled, v, out)
        # the rows of y are rounded to bfloat16 before the product, by either way of doing the norm
        unfused = torch.empty(m, hidden, dtype=torch.bfloat16, device=DEV)
        ops.rmsnorm(x, gain, eps, unfused)
        by_the_kernel = unfused.double().cpu() @ plain_v.double().cpu().t()
        spread = rel(by_the_kernel, want)
        ulps = ULP["bfloat16" if out_dtype == torch.bfloat16 else "float32"] * 2
        assert rel(out.cpu(), want) < 2 * spread + ulps
        if small is not None:                                   # compared alone: the error's scale is the row's own
            assert rel(out[small].cpu(), want[small]) < 2 * rel(by_the_kernel[small], want[small]) + ulps
            assert float(out[zero].abs().max()) == 0.0
    glu = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    ops.linear_glu(scaled, v_glu, glu)
    assert rel(glu.cpu(), P.swiglu(want[:, :n], want[:, n:])) < 2e-2
    if small is not None:
        assert rel(glu[small].cpu(), P.swiglu(want[small, :n], want[small, n:])) < 2e-2
        assert float(glu[zero].abs().max()) == 0.0
    # and once more into the residual stream, with the norm after it handed on again
    again = ops.linear(scaled, packed_or_not(ops, plain_v[:hidden % 64 + 64].contiguous(), packed),
                       torch.zeros(m, hidden % 64 + 64, device=DEV), accumulate=True,
                       then_norm=((rand(hidden % 64 + 64, seed=6) + 1.0), eps))
    assert (again is not None) == (m <= 16)                     # 64 to 127 columns: only the kernel for up to 16 rows writes them


@pytest.mark.parametrize("m,hidden,k", [(520, 1032, 4160), (2048, 4096, 4096), (600, 520, 8192), (1024, 8192, 4096)])
@pytest.mark.parametrize("gain_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("packed", [False, True])
def test_rmsnorm_done_by_the_second_kernel_of_a_product_of_many_rows(ops, m, hidden, k, gain_dtype, packed):
    # x += a w^T; y = rmsnorm(x) * gain: with many rows, few columns and a long k the product runs as large tiles that split
    # k, and the kernel that adds the parts writes y as well: the norm kernel's result to the bit
    a = rand(m, k, dtype=torch.bfloat16, seed=1)
    w = rand(hidden, k, dtype=torch.bfloat16, seed=2, scale=0.1)
    x = rand(m, hidden, seed=3, scale=2.0)
    x[m // 2] *= 50.0
    eps = 1e-3
    a[0], a[m - 1] = 0.0, 0.0                                   # a row whose mean square is about eps, and a row of zeros
    x[0], x[m - 1] = rand(hidden, seed=7, scale=0.03), 0.0
    gain = (rand(hidden, seed=4) + 1.0).to(gain_dtype)
    fresh = x.double().cpu() + a.double().cpu() @ w.double().cpu().t()
    alone = x.clone()
    w = packed_or_not(ops, w, packed)
    normed = ops.linear(a, w, x, accumulate=True, then_norm=(gain, eps))
    assert isinstance(normed, torch.Tensor) and normed.dtype == torch.bfloat16 and normed.shape == (m, hidden)
    assert rel(x.cpu(), fresh) < 1e-5
    assert ops.linear(a, w, alone, accumulate=True) is None
    assert rel(alone.cpu(), fresh) < 1e-5
    by_the_norm_kernel = torch.empty(m, hidden, dtype=torch.bfloat16, device=DEV)
    ops.rmsnorm(x, gain, eps, by_the_norm_kernel)
    assert torch.equal(normed, by_the_norm_kernel)
    want = P.rmsnorm(fresh, gain.double().cpu(), eps)
    assert rel(normed.cpu(), want) < ULP["bfloat16"]
    assert rel(normed[0].cpu(), want[0]) < ULP["bfloat16"]      # eps counts here, once and inside the root
    assert float(normed[m - 1].abs().max()) == 0.0


def test_rmsnorm_is_left_to_its_own_kernel_where_the_products_cannot_do_it(ops):
    gain = rand(200, seed=4).to(torch.bfloat16)
    for m, dtype in ((17, torch.bfloat16), (300, torch.bfloat16), (4, torch.float32)):
        a, w = rand(m, 64, dtype=dtype), rand(200, 64, dtype=dtype)
        x = rand(m, 200, seed=3)
        want = x.double().cpu() + a.double().cpu() @ w.double().cpu().t()
        assert ops.linear(a, w, x, accumulate=True, then_norm=(gain, 1e-5)) is None
        assert rel(x.cpu(), want) < 1e-5
    assert ops.linear(rand(4, 64, dtype=torch.bfloat16), rand(204, 64, dtype=torch.bfloat16), rand(4, 204),
                      accumulate=True, then_norm=(rand(204).to(torch.bfloat16), 1e-5)) is None   # 204 columns: no product takes them


def test_linear_refuses_what_it_cannot_do(ops):
    from xeno_rt_amd.ops.hip import KernelError
    a, w = rand(2, 8), rand(4, 8)
    with pytest.raises(KernelError, match="columns"):
        ops.linear(a, rand(4, 16), torch.empty(2, 4, device=DEV))
    with pytest.raises(KernelError, match="shape"):
        ops.linear(a, w, torch.empty(2, 5, device=DEV))
    with pytest.raises(KernelError, match="float32 output"):
        ops.linear(a, w, torch.empty(2, 4, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(KernelError, match="contiguous"):
        ops.linear(rand(8, 2).t(), w, torch.empty(2, 4, device=DEV))
    with pytest.raises(KernelError, match="GPU"):
        ops.linear(a.cpu(), w, torch.empty(2, 4, device=DEV))
    # the gated product's activation: a name the package does not know, a code the library does not know
    with pytest.raises(KernelError, match="activation"):
        ops.linear_glu(a, w, torch.empty(2, 2, device=DEV), activation="gelu")
    for operands in ((a, w), (rand(2, 64, dtype=torch.bfloat16), rand(32, 64, dtype=torch.bfloat16))):   # every kernel's entry
        with pytest.raises(KernelError, match="unknown activation 3"):
            ops._linear(*operands, torch.empty(2, operands[1].shape[0] // 2, dtype=operands[0].dtype, device=DEV),
                        2 | (3 << 8), operands[1].shape[0] // 2)
    with pytest.raises(KernelError, match="unknown activation"):
        ops._linear(a, w, torch.empty(2, 4, device=DEV), 0 | (1 << 8), 4)        # only a gated product has one


def test_attention_refuses_values_of_another_width_than_the_keys(ops):
    from xeno_rt_amd.ops.hip import KernelError
    kv = make_cache(4, 2, 32, torch.float32, 1, 4)
    kv.v = torch.zeros(4, 2, 48, 64, device=DEV)
    qkv = rand(3, (4 + 2 * 2) * 32)
    batch = SimpleNamespace(positions=i32([0, 1, 2]), slots=i32([0, 0, 0]))
    with pytest.raises(KernelError, match="as wide as the keys"):
        ops.attention(qkv, 4, 2, 32, kv, batch, torch.empty(3, 4 * 32, device=DEV), scale=1.0)


# ---- q/k/v preparation and attention ------------------------------------------------------

def make_cache(n_blocks, nkv, hd, dtype, slots, max_blocks):
    k = torch.zeros(n_blocks, nkv, 64, hd, dtype=dtype, device=DEV)
    v = torch.zeros(n_blocks, nkv, hd, 64, dtype=dtype, device=DEV)
    table = torch.full((slots, max_blocks), -1, dtype=torch.int32, device=DEV)
    return SimpleNamespace(k=k, v=v, block_table=table)


def clone_cache(kv):
    return SimpleNamespace(k=kv.k.clone(), v=kv.v.clone(), block_table=kv.block_table.clone())


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd,rope_dim", [(4, 2, 16, 16), (6, 3, 32, 32), (8, 1, 128, 128),
                                                (5, 5, 48, 48), (2, 1, 256, 256), (4, 4, 64, 32),
                                                (4, 2, 100, 100), (3, 3, 72, 72), (2, 1, 10, 10), (2, 2, 6, 4)])
def test_qkv_prepare(ops, dtype, nh, nkv, hd, rope_dim):
    tokens = 9
    qkv = rand(tokens, (nh + 2 * nkv) * hd, dtype=DT[dtype], seed=hd)
    qkv[1] *= 0.01                   # heads whose mean square is about the norm's eps: eps decides their scale
    qkv[2] = 0.0                     # and heads of zeros, which stay zeros
    positions = i32([0, 1, 63, 64, 65, 127, 128, 500, 1000])
    slots = i32([0, 0, 0, 0, 1, 1, -1, 1, 0])                  # one token is padding
    kv = make_cache(40, nkv, hd, DT[dtype], 2, 16)
    kv.block_table[0, :16] = torch.arange(3, 19, dtype=torch.int32)
    kv.block_table[1, :16] = torch.arange(39, 23, -1, dtype=torch.int32)
    theta = (torch.tensor(10000.0) ** (torch.arange(rope_dim // 2) * 2.0 / rope_dim)).to(DEV)
    qn, kn = rand(hd, seed=1) + 1.0, rand(hd, seed=2) + 1.0
    for norms in (False, True):
        got, want = qkv.clone(), qkv.clone()
        kv_got, kv_want = clone_cache(kv), clone_cache(kv)
        args = dict(q_norm=qn if norms else None, k_norm=kn if norms else None, norm_eps=1e-4,
                    rope_theta=theta, rope_dim=rope_dim, rope_scale=1.0)
        ops.qkv_prepare(got, nh, nkv, hd, positions, slots, kv=kv_got, **args)
        REF.qkv_prepare(want, nh, nkv, hd, positions, slots, kv=kv_want, **args)
        # sine and cosine of angles up to 1000 rad differ by float32 rounding of the angle
        tol = 3e-5 if dtype == "float32" else ULP[dtype]
        assert rel(got.float(), want.float()) < tol
        assert rel(kv_got.k.float(), kv_want.k.float()) < tol
        assert torch.equal(kv_got.v, kv_want.v)
        assert int((cache_order.plain_keys(kv_got.k) != 0).any(-1).sum()) == 7 * nkv      # seven tokens cached: not the padding, and not the zeros
        assert float(got[2].abs().max()) == 0.0
        # the small token alone, against the plain formulas (norm of every head, then the rotation) in 64-bit
        q = qkv[1:2, :nh * hd].double().cpu()
        if norms:
            q = P.head_rmsnorm(q, nh, hd, qn.double().cpu(), 1e-4)
        q = P.rope(q, nh, hd, torch.tensor([1]), rope_dim, 10000.0)
        assert rel(got[1, :nh * hd].float().cpu(), q[0]) < (5e-6 if dtype == "float32" else ULP[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd,rope_dim", [(4, 2, 128, 128), (3, 3, 64, 64), (2, 1, 256, 256), (4, 2, 48, 48),
                                                (4, 2, 64, 16)])
def test_qkv_prepare_of_many_tokens(ops, dtype, nh, nkv, hd, rope_dim):
    """A prefill step: three sequences, one of which continues in the middle of a cache block, one padding
    token between them; the values reach their transposed blocks through the kernel that turns tiles."""
    runs = [(0, 0, 70), (1, 37, 100), (-1, 0, 1), (2, 64, 30)]          # slot, first position, tokens
    slots = [slot for slot, _, count in runs for _ in range(count)]
    positions = [first + i for _, first, count in runs for i in range(count)]
    tokens = len(slots)
    qkv = rand(tokens, (nh + 2 * nkv) * hd, dtype=DT[dtype], seed=hd + 1)
    kv = make_cache(40, nkv, hd, DT[dtype], 3, 4)
    kv.block_table[0, :4] = i32([7, 3, 11, 2])
    kv.block_table[1, :4] = i32([30, 31, 5, 6])
    kv.block_table[2, :4] = i32([20, 19, 18, 17])
    theta = (torch.tensor(10000.0) ** (torch.arange(rope_dim // 2) * 2.0 / rope_dim)).to(DEV)
    qn, kn = rand(hd, seed=1) + 1.0, rand(hd, seed=2) + 1.0
    got, want = qkv.clone(), qkv.clone()
    kv_got, kv_want = clone_cache(kv), clone_cache(kv)
    args = dict(q_norm=qn, k_norm=kn, norm_eps=1e-4, rope_theta=theta, rope_dim=rope_dim, rope_scale=1.0)
    ops.qkv_prepare(got, nh, nkv, hd, i32(positions), i32(slots), kv=kv_got, longest_run=100, **args)
    REF.qkv_prepare(want, nh, nkv, hd, i32(positions), i32(slots), kv=kv_want, **args)
    tol = 3e-5 if dtype == "float32" else ULP[dtype]
    assert rel(got.float(), want.float()) < tol
    assert rel(kv_got.k.float(), kv_want.k.float()) < tol
    assert torch.equal(kv_got.v, kv_want.v)
    assert int((cache_order.plain_keys(kv_got.k) != 0).any(-1).sum()) == (tokens - 1) * nkv


@pytest.mark.parametrize("nh,nkv,hd,rope_dim,k,tokens", [(32, 8, 128, 128, 4096, 8), (4, 2, 64, 64, 200, 9), (3, 3, 48, 32, 96, 16),
                                                          (2, 1, 256, 256, 72, 1), (5, 1, 16, 16, 64, 3), (4, 2, 64, 0, 128, 9),
                                                          (4, 4, 80, 48, 264, 7),
                                                          # 17 to 64 tokens: the product is split along k, and the kernel that
                                                          # adds the partial sums does the rest (the third: two kernels)
                                                          (32, 8, 128, 128, 4096, 40), (4, 2, 64, 64, 256, 17),
                                                          (3, 3, 48, 32, 192, 33), (4, 2, 64, 0, 128, 64), (6, 2, 96, 96, 320, 64)])
@pytest.mark.parametrize("packed", [False, True])
def test_linear_qkv_in_one_kernel(ops, nh, nkv, hd, rope_dim, k, tokens, packed):
    """The projection of a short step with the rotation and the cache write in its epilogue, against the two
    kernels one after the other; without a norm before it and with one."""
    positions = ([0, 1, 63, 64, 65, 127, 128, 500, 1000, 2, 3, 4, 5, 6, 7, 8] + list(range(9, 57)))[:tokens]
    slots = ([0, 0, 0, 0, 1, 1, -1, 1, 0, 1, 1, 1, 1, 1, 1, 1] + [0] * 48)[:tokens]                # one token is padding
    positions, slots = i32(positions), i32(slots)
    width = (nh + 2 * nkv) * hd
    a = rand(tokens, k, dtype=torch.bfloat16, seed=hd)
    w = rand(width, k, dtype=torch.bfloat16, seed=k, scale=1.0 / math.sqrt(k))
    kv = make_cache(40, nkv, hd, torch.bfloat16, 2, 16)
    kv.block_table[0, :16] = torch.arange(3, 19, dtype=torch.int32)
    kv.block_table[1, :16] = torch.arange(39, 23, -1, dtype=torch.int32)
    theta = (torch.tensor(10000.0) ** (torch.arange(rope_dim // 2) * 2.0 / max(rope_dim, 1))).to(DEV) if rope_dim else None
    args = dict(rope_theta=theta, rope_dim=rope_dim, rope_scale=0.5)
    # the norm before the projection, handed over by the product before it
    x = rand(tokens, k, seed=3, scale=2.0)
    gain = (rand(k, seed=4) + 1.0).to(torch.bfloat16)
    inner = 64 if tokens <= 16 else 256
    before = rand(tokens, inner, dtype=torch.bfloat16, seed=5)
    if tokens >= 3:                  # a row whose mean square is about the norm's eps, and a row of zeros
        before[1], before[2] = 0.0, 0.0
        x[1], x[2] = rand(k, seed=8, scale=0.01), 0.0
    scaled = ops.linear(before, rand(k, inner, dtype=torch.bfloat16, seed=6), x, accumulate=True, then_norm=(gain, 1e-4))
    assert scaled is not None
    normed_small = P.rmsnorm(x[1:2].double().cpu(), gain.double().cpu(), 1e-4) if tokens >= 3 else None
    # packed as the attention part packs it: the pairs of a rotation over whole heads side by side
    plain_w = w
    w = packed_or_not(ops, w, packed, "rotary", head_dim=hd, rotated_heads=nh + nkv if rope_dim == hd else 0)
    for rows in (a, scaled):
        got = torch.empty(tokens, width, dtype=torch.bfloat16, device=DEV)
        want = torch.empty(tokens, width, dtype=torch.bfloat16, device=DEV)
        kv_got, kv_want = clone_cache(kv), clone_cache(kv)
        ops.linear_qkv(rows, w, got, nh, nkv, hd, positions, slots, kv=kv_got, **args)
        ops.linear(rows, plain_w, want)
        ops.qkv_prepare(want, nh, nkv, hd, positions, slots, kv=kv_want, **args)
        # the same sums, roundings and formulas in both: at most the contraction of a multiply-add may differ
        assert rel(got.float(), want.float()) < ULP["bfloat16"]
        assert float((got.float() - want.float()).abs().gt(0).float().mean()) < 0.01
        assert rel(kv_got.k.float(), kv_want.k.float()) < ULP["bfloat16"]
        assert torch.equal(kv_got.v, kv_want.v)
        zeros = 1 if rows is scaled and tokens >= 3 else 0       # the row of zeros is cached as zeros
        assert int((cache_order.plain_keys(kv_got.k) != 0).any(-1).sum()) == (int((slots >= 0).sum()) - zeros) * nkv
        if rows is scaled and tokens >= 3:
            # the small row alone against the plain formulas: its scale hangs on the eps of the norm before the projection
            assert float(got[2].abs().max()) == 0.0
            q = (normed_small @ plain_w[:nh * hd].double().cpu().t())
            q = P.rope(q, nh, hd, torch.tensor([int(positions[1])]), rope_dim, 10000.0, scale=0.5) if rope_dim else q
            assert rel(got[1, :nh * hd].float().cpu(), q[0]) < 1e-2
    # without a cache to write (a layer that reads another layer's), and with head norms (two kernels then)
    got = torch.empty(tokens, width, dtype=torch.bfloat16, device=DEV)
    want = torch.empty(tokens, width, dtype=torch.bfloat16, device=DEV)
    ops.linear_qkv(a, w, got, nh, nkv, hd, positions, slots, **args)
    ops.linear(a, plain_w, want)
    ops.qkv_prepare(want, nh, nkv, hd, positions, slots, **args)
    assert rel(got.float(), want.float()) < ULP["bfloat16"]
    qn, kn = rand(hd, seed=1) + 1.0, rand(hd, seed=2) + 1.0
    kv_got, kv_want = clone_cache(kv), clone_cache(kv)
    ops.linear_qkv(a, w, got, nh, nkv, hd, positions, slots, q_norm=qn, k_norm=kn, norm_eps=1e-4, kv=kv_got, **args)
    ops.linear(a, w, want)
    ops.qkv_prepare(want, nh, nkv, hd, positions, slots, q_norm=qn, k_norm=kn, norm_eps=1e-4, kv=kv_want, **args)
    assert torch.equal(got, want) and torch.equal(kv_got.k, kv_want.k) and torch.equal(kv_got.v, kv_want.v)
    if packed:          # and the packed projection alone against the plain one
        ops.linear(a, w, want)
        ops.linear(a, plain_w, got)
        assert rel(want.float(), got.float()) < ULP["bfloat16"] * 2


def test_rope_reference_vector_and_pairing(ops):
    # tests/kernels_test.rs:94-108: one head of 4, position 2, base 1e4 -> pairs (0,2), (1,3)
    qkv = torch.zeros(1, 3 * 16, device=DEV)
    qkv[0, :4] = torch.tensor([1.0, 2.0, 3.0, 4.0])
    theta = torch.tensor([1.0, 100.0], device=DEV)
    ops.qkv_prepare(qkv, 1, 1, 16, i32([2]), i32([-1]), rope_theta=theta, rope_dim=4)
    a0, a1 = 2.0, 0.02
    want = torch.tensor([1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
                         1 * math.sin(a0) + 3 * math.cos(a0), 2 * math.sin(a1) + 4 * math.cos(a1)])
    assert rel(qkv[0, :4].cpu(), want) < 1e-6
    assert float(qkv[0, 4:].abs().max()) == 0.0                   # beyond rope_dim nothing moves


def filled_cache(nkv, hd, dtype, lengths, seed=0):
    """A cache holding `lengths[s]` random tokens for slot s, blocks deliberately out of order."""
    max_blocks = max((n + 63) // 64 for n in lengths) + 1
    n_blocks = len(lengths) * max_blocks + 3
    kv = make_cache(n_blocks, nkv, hd, dtype, len(lengths), max_blocks)
    order = torch.randperm(n_blocks, generator=torch.Generator().manual_seed(seed)).tolist()
    keys, values = [], []
    for s, n in enumerate(lengths):
        k = rand(n, nkv, hd, dtype=dtype, seed=seed + 10 * s + 1)
        v = rand(n, nkv, hd, dtype=dtype, seed=seed + 10 * s + 2)
        keys.append(k); values.append(v)
        for b in range((n + 63) // 64):
            block = order.pop()
            kv.block_table[s, b] = block
            part = slice(b * 64, min(n, b * 64 + 64))
            kv.k[block, :, :part.stop - part.start, :] = k[part].transpose(0, 1)
            kv.v[block, :, :, :part.stop - part.start] = v[part].permute(1, 2, 0)
    # what lies beyond a sequence's end must never be read: poison it
    for s, n in enumerate(lengths):
        if n % 64:
            block = int(kv.block_table[s, n // 64])
            kv.k[block, :, n % 64:, :] = float("nan")
            kv.v[block, :, :, n % 64:] = float("nan")
    kv.k, kv.v = cache_order.store_keys(kv.k), cache_order.store_values(kv.v)     # from rows into the order the kernels keep
    return kv, keys, values


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd", [(4, 2, 16), (6, 3, 32), (8, 1, 128), (5, 5, 48), (2, 2, 256), (32, 8, 128),
                                       (4, 2, 100), (3, 3, 72), (2, 1, 10), (4, 2, 6)])
def test_attention(ops, dtype, nh, nkv, hd):
    lengths = [200, 65, 1]
    kv, keys, values = filled_cache(nkv, hd, DT[dtype], lengths, seed=hd)
    # queries: the last tokens of every sequence (a prompt's end), some in the middle, one padding
    slots = [0, 0, 0, 0, 1, 1, 2, -1, 0]
    positions = [199, 198, 64, 0, 64, 63, 0, 0, 127]
    qkv = rand(len(slots), (nh + 2 * nkv) * hd, dtype=DT[dtype], seed=7)
    batch = SimpleNamespace(slots=i32(slots), positions=i32(positions))
    out = torch.full((len(slots), nh * hd), 7.0, dtype=DT[dtype], device=DEV)
    scale = 1.0 / math.sqrt(hd)
    ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=scale)
    for t, (slot, pos) in enumerate(zip(slots, positions)):
        if slot < 0:
            assert float(out[t].abs().max()) == 0.0
            continue
        q = qkv[t:t + 1, :nh * hd].double().cpu()
        k = keys[slot][:pos + 1].reshape(pos + 1, nkv * hd).double().cpu()
        v = values[slot][:pos + 1].reshape(pos + 1, nkv * hd).double().cpu()
        want = P.causal_attention(q, k, v, nh, nkv, hd, start_position=pos)
        assert rel(out[t:t + 1].cpu(), want) < (2e-5 if dtype == "float32" else 1e-2), (t, slot, pos)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 48, None), (8, 2, 128, None), (2, 1, 100, None), (4, 4, 32, 700)])
def test_general_attention_gives_the_same_bits_with_few_tokens_and_with_many(ops, dtype, nh, nkv, hd, window):
    """The general kernel takes a step of few tokens with a workgroup of wavefronts per (token, head), which work the
    chunks of keys off side by side, and a step of many tokens with one wavefront each, which takes the chunks one after
    the other, and there two or four query heads of a key/value head together (groups of 2 and 4 here): the same sums in
    the same order. Sequences of one, two and six chunks of 512 keys, some ending inside a chunk; the same queries alone
    and among 3000 others."""
    lengths = [3000, 513, 512, 70, 1025]
    kv, keys, values = filled_cache(nkv, hd, DT[dtype], lengths, seed=hd)
    slots = [0, 1, 2, 3, 4, 0, 0, 4]
    positions = [2999, 512, 511, 69, 1024, 1536, 600, 1023]
    few = rand(len(slots), (nh + 2 * nkv) * hd, dtype=DT[dtype], seed=7)
    out_few = torch.empty(len(slots), nh * hd, dtype=DT[dtype], device=DEV)
    ops.attention(few, nh, nkv, hd, kv, SimpleNamespace(slots=i32(slots), positions=i32(positions)), out_few,
                  scale=1.0 / math.sqrt(hd), window=window)
    crowd = 3000                                               # other tokens of the step: early positions of sequence 0
    many = torch.cat([rand(crowd, (nh + 2 * nkv) * hd, dtype=DT[dtype], seed=8), few])
    out_many = torch.empty(crowd + len(slots), nh * hd, dtype=DT[dtype], device=DEV)
    batch = SimpleNamespace(slots=i32([0] * crowd + slots), positions=i32([t % 64 for t in range(crowd)] + positions))
    ops.attention(many, nh, nkv, hd, kv, batch, out_many, scale=1.0 / math.sqrt(hd), window=window)
    assert torch.isfinite(out_few).all()
    assert torch.equal(out_many[crowd:], out_few)
    for t, (slot, pos) in enumerate(zip(slots, positions)):    # and both are the plain attention's
        if window is not None:
            continue
        q = few[t:t + 1, :nh * hd].double().cpu()
        k = keys[slot][:pos + 1].reshape(pos + 1, nkv * hd).double().cpu()
        v = values[slot][:pos + 1].reshape(pos + 1, nkv * hd).double().cpu()
        want = P.causal_attention(q, k, v, nh, nkv, hd, start_position=pos)
        assert rel(out_few[t:t + 1].cpu(), want) < (2e-5 if dtype == "float32" else 1e-2), (t, slot, pos)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_finds_a_far_key(ops, dtype):
    """One key among 900 matches the query: the output must be that key's value, wherever it lies."""
    nh, nkv, hd = 4, 2, 64
    kv, keys, values = filled_cache(nkv, hd, DT[dtype], [900], seed=1)
    for far in (0, 5, 63, 64, 500, 899):
        qkv = torch.zeros(1, (nh + 2 * nkv) * hd, dtype=DT[dtype], device=DEV)
        for head in range(nh):
            qkv[0, head * hd:(head + 1) * hd] = keys[0][far, head // 2] * 40.0
        batch = SimpleNamespace(slots=i32([0]), positions=i32([899]))
        out = torch.empty(1, nh * hd, dtype=DT[dtype], device=DEV)
        ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
        for head in range(nh):
            got = out[0, head * hd:(head + 1) * hd].float()
            assert rel(got, values[0][far, head // 2].float()) < 2e-2, (far, head)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd", [(6, 3, 32), (8, 2, 128)])
def test_attention_with_scores_biased_by_distance(ops, cpp, dtype, nh, nkv, hd):
    """distance_slopes: a key at position j adds slope * (j - P) to the scaled score of the query at P, one slope per
    query head (also where the matrix-core kernels would run without it: a described decode step and a prefill).
    Against float64 on the host and against the plain C++ reference."""
    lengths = [200, 65]
    kv, keys, values = filled_cache(nkv, hd, DT[dtype], lengths, seed=hd + 1)
    slopes = torch.tensor([0.5 ** (h + 1) for h in range(nh)], dtype=torch.float32, device=DEV)
    scale = 1.0 / math.sqrt(hd)
    for batch, slots, positions in (
            (SimpleNamespace(slots=i32([0, 0, 1, -1]), positions=i32([199, 64, 64, 0])), [0, 0, 1, -1], [199, 64, 64, 0]),
            (described([0, 1], [1, 1], [199, 64]), [0, 1], [199, 64]),
            (described([0], [40], [160]), [0] * 40, list(range(160, 200)))):
        qkv = rand(len(slots), (nh + 2 * nkv) * hd, dtype=DT[dtype], seed=9)
        out = torch.full((len(slots), nh * hd), 7.0, dtype=DT[dtype], device=DEV)
        ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=scale, distance_slopes=slopes)
        plain = torch.empty_like(out)
        ops.attention(qkv, nh, nkv, hd, kv, batch, plain, scale=scale)
        from_cpp = cpp.attention(qkv.cpu(), nh, nkv, hd, kv.k.cpu(), kv.v.cpu(), kv.block_table.cpu(), torch.tensor(positions), torch.tensor(slots), scale,
                                 distance_slopes=slopes.cpu())
        for t, (slot, pos) in enumerate(zip(slots, positions)):
            if slot < 0:
                assert float(out[t].abs().max()) == 0.0
                continue
            k = keys[slot][:pos + 1].double().cpu()                 # [keys, kv heads, dim]
            v = values[slot][:pos + 1].double().cpu()
            distance = torch.arange(pos + 1, dtype=torch.float64) - pos
            want = torch.empty(nh * hd, dtype=torch.float64)
            for head in range(nh):
                q = qkv[t, head * hd:(head + 1) * hd].double().cpu()
                scores = (k[:, head // (nh // nkv)] @ q) * scale + float(slopes[head]) * distance
                want[head * hd:(head + 1) * hd] = torch.softmax(scores, 0) @ v[:, head // (nh // nkv)]
            limit = 2e-5 if dtype == "float32" else 1e-2
            assert rel(out[t].cpu(), want) < limit, (t, slot, pos)
            assert rel(from_cpp[t], want) < 2e-5, (t, slot, pos)
            if pos > 8:
                assert rel(plain[t].cpu(), want) > 10 * limit        # the slopes do change the result


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_window_edge(ops, dtype):
    """With a window of W a query at P sees keys P-W+1..P: a loud key just outside must be
    ignored, the same key just inside must win."""
    nh, nkv, hd, window = 2, 1, 32, 100
    kv, keys, values = filled_cache(nkv, hd, DT[dtype], [400], seed=2)
    pos = 399
    for key_at, inside in ((300, True), (299, False)):
        qkv = torch.zeros(1, (nh + 2 * nkv) * hd, dtype=DT[dtype], device=DEV)
        for head in range(nh):
            qkv[0, head * hd:(head + 1) * hd] = keys[0][key_at, 0] * 40.0
        batch = SimpleNamespace(slots=i32([0]), positions=i32([pos]))
        out = torch.empty(1, nh * hd, dtype=DT[dtype], device=DEV)
        ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd), window=window)
        ref = torch.empty(1, nh * hd, dtype=DT[dtype], device=DEV)
        REF.attention(qkv, nh, nkv, hd, kv, batch, ref, 1.0 / math.sqrt(hd), window=window)
        assert rel(out.float(), ref.float()) < (2e-5 if dtype == "float32" else 1e-2)
        hit = rel(out[0, :hd].float(), values[0][key_at, 0].float()) < 2e-2
        assert hit == inside


def described(slots, counts, starts):
    """A batch namespace with the per-sequence arrays, as the engine builds it."""
    token_slots, positions, offsets = [], [], [0]
    for slot, count, start in zip(slots, counts, starts):
        token_slots += [slot] * count
        positions += list(range(start, start + count))
        offsets.append(offsets[-1] + count)
    return SimpleNamespace(slots=i32(token_slots), positions=i32(positions), sequence_offsets=i32(offsets),
                           sequence_slots=i32(slots), sequence_starts=i32(starts), n_sequences=len(slots),
                           max_count=max(counts), max_context=max(s + c for s, c in zip(starts, counts)))


def expected_attention(qkv, batch_slots, batch_positions, keys, values, nh, nkv, hd):
    rows = []
    for t, (slot, pos) in enumerate(zip(batch_slots, batch_positions)):
        q = qkv[t:t + 1, :nh * hd].double().cpu()
        k = keys[slot][:pos + 1].reshape(pos + 1, nkv * hd).double().cpu()
        v = values[slot][:pos + 1].reshape(pos + 1, nkv * hd).double().cpu()
        rows.append(P.causal_attention(q, k, v, nh, nkv, hd, start_position=pos))
    return torch.cat(rows)


@pytest.mark.parametrize("nh,nkv,hd", [(4, 4, 64), (8, 2, 128), (32, 8, 128), (16, 1, 64), (40, 2, 128)])
def test_attention_decode_on_matrix_cores(ops, nh, nkv, hd):
    """One token per sequence (the decode kernels): lengths at block edges, one sequence far longer
    than the others, groups of 1 to 20 query heads per key/value head."""
    lengths = [1, 64, 65, 700, 128, 2]
    kv, keys, values = filled_cache(nkv, hd, torch.bfloat16, lengths, seed=hd + nh)
    slots = list(range(len(lengths)))
    batch = described(slots, [1] * len(lengths), [n - 1 for n in lengths])
    qkv = rand(len(lengths), (nh + 2 * nkv) * hd, dtype=torch.bfloat16, seed=3)
    out = torch.full((len(lengths), nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
    want = expected_attention(qkv, slots, [n - 1 for n in lengths], keys, values, nh, nkv, hd)
    assert torch.isfinite(out).all()
    assert rel(out.cpu(), want) < 1e-2
    # a padded batch: the extra token has no slot and gets zeros, the others do not change
    padded = SimpleNamespace(**vars(batch))
    padded.slots, padded.positions = i32(slots + [-1]), i32([n - 1 for n in lengths] + [0])
    out2 = torch.full((len(lengths) + 1, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention(torch.cat([qkv, qkv[:1]]), nh, nkv, hd, kv, padded, out2, scale=1.0 / math.sqrt(hd))
    assert torch.equal(out2[:-1], out) and float(out2[-1].abs().max()) == 0.0


@pytest.mark.parametrize("norms", [True, False])
@pytest.mark.parametrize("rotated", [True, False])
@pytest.mark.parametrize("nh,nkv,hd", [(4, 4, 64), (8, 2, 128), (32, 8, 128), (64, 8, 128), (40, 2, 128)])
def test_attention_decode_that_finishes_q_k_and_v_itself(ops, nh, nkv, hd, rotated, norms):
    """A decode step in which the attention kernel does what qkv_prepare would have done before it (head norms,
    rotation, cache write of the new key and value), against the two kernels one after the other: the same
    formulas, so the results agree to the rounding of bfloat16. Sequences whose newest token is the first of all,
    the first and the last of a block, and far out (several parts of keys); one padding token."""
    from xeno_rt_amd.ops.hip import QkvFinish
    lengths = [1, 64, 65, 700, 128, 2, 1500]
    kv, keys, values = filled_cache(nkv, hd, torch.bfloat16, lengths, seed=hd + nh)
    # the newest token's place in the cache holds what an earlier sequence left there: both ways must overwrite it
    slots = list(range(len(lengths)))
    positions = [n - 1 for n in lengths]
    batch = described(slots + [-1], [1] * (len(lengths) + 1), positions + [0])
    batch.slots, batch.positions = i32(slots + [-1]), i32(positions + [0])
    tokens = len(lengths) + 1
    raw = rand(tokens, (nh + 2 * nkv) * hd, dtype=torch.bfloat16, seed=3)
    raw[3] *= 0.02                                          # heads whose mean square is about the norm's eps
    theta = (torch.tensor(10000.0) ** (torch.arange(hd // 2) * 2.0 / hd)).to(DEV) if rotated else None
    qn, kn = (rand(hd, seed=1) + 1.0, rand(hd, seed=2) + 1.0) if norms else (None, None)
    args = dict(q_norm=qn, k_norm=kn, norm_eps=1e-4, rope_theta=theta, rope_dim=hd if rotated else 0, rope_scale=0.5)
    scale = 1.0 / math.sqrt(hd)
    table = ops.rope_table(theta, hd, 0.5, 1500) if rotated else None      # cosines and sines of the positions' angles, made once
    assert ops.attention_finishes_qkv(torch.bfloat16, nh, nkv, hd, batch, None, args["rope_dim"], table)
    if rotated:
        assert not ops.attention_finishes_qkv(torch.bfloat16, nh, nkv, hd, batch, None, hd, table[:1499])   # a position beyond the table
        angles = torch.arange(1500, dtype=torch.float32)[:, None] * 0.5 / theta.cpu()[None, :]
        assert rel(table[..., 0].cpu(), torch.cos(angles.double())) < 1e-4 and rel(table[..., 1].cpu(), torch.sin(angles.double())) < 1e-4
    # the two kernels
    kv_two, qkv_two = clone_cache(kv), raw.clone()
    ops.qkv_prepare(qkv_two, nh, nkv, hd, batch.positions, batch.slots, kv=kv_two, **args)
    out_two = torch.full((tokens, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention(qkv_two, nh, nkv, hd, kv_two, batch, out_two, scale=scale)
    # the one
    kv_one, qkv_one = clone_cache(kv), raw.clone()
    out_one = torch.full((tokens, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention(qkv_one, nh, nkv, hd, kv_one, batch, out_one, scale=scale, finish=QkvFinish(qn, kn, 1e-4, table))
    assert torch.equal(qkv_one, raw)                        # q, k and v stay as the projection left them
    assert torch.isfinite(out_one).all() and float(out_one[-1].abs().max()) == 0.0
    assert rel(out_one[:-1].float(), out_two[:-1].float()) < 1e-2
    for row in range(tokens - 1):                           # every sequence by itself: short ones are not hidden by long ones
        assert rel(out_one[row].float(), out_two[row].float()) < 2e-2, row
    # (what lies beyond the sequences' ends is poisoned with NaN in both caches and stays so)
    assert torch.equal(torch.nan_to_num(kv_one.v.float(), nan=123.0), torch.nan_to_num(kv_two.v.float(), nan=123.0))
    plain_one, plain_two = cache_order.plain_keys(kv_one.k).float(), cache_order.plain_keys(kv_two.k).float()
    same = torch.nan_to_num(plain_one, nan=123.0) == torch.nan_to_num(plain_two, nan=123.0)
    close = (plain_one - plain_two).abs() <= ULP["bfloat16"] * plain_two.abs().clamp(min=1e-3) * 2
    assert bool((same | close).all())
    assert float(same.float().mean()) > 0.999               # only the newest keys can differ at all, by a rounding


@pytest.mark.parametrize("nh,nkv,hd", [(32, 8, 128), (24, 8, 64)])
def test_attention_decode_of_many_sequences(ops, nh, nkv, hd):
    """Seventy sequences: with so many (sequence, key/value head) pairs a workgroup takes all keys of its pair
    and writes the result itself, without partial results and a merge; padding still gets zeros."""
    lengths = [1 + (37 * i) % 300 for i in range(69)] + [900]
    kv, keys, values = filled_cache(nkv, hd, torch.bfloat16, lengths, seed=hd)
    slots = list(range(len(lengths)))
    positions = [n - 1 for n in lengths]
    batch = described(slots + [-1], [1] * (len(lengths) + 1), positions + [0])
    batch.slots, batch.positions = i32(slots + [-1]), i32(positions + [0])
    qkv = rand(len(lengths) + 1, (nh + 2 * nkv) * hd, dtype=torch.bfloat16, seed=3)
    out = torch.full((len(lengths) + 1, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
    want = expected_attention(qkv[:-1], slots, positions, keys, values, nh, nkv, hd)
    assert torch.isfinite(out).all()
    assert rel(out[:-1].cpu(), want) < 1e-2
    assert float(out[-1].abs().max()) == 0.0


@pytest.mark.parametrize("nh,nkv,hd", [(4, 4, 64), (8, 2, 128), (32, 8, 128), (6, 3, 64)])
def test_attention_prefill_on_matrix_cores(ops, nh, nkv, hd):
    """Whole prompts of unequal lengths in one step, and a prompt that continues a cache."""
    lengths = [200, 65, 1, 33, 500]
    starts = [0, 0, 0, 20, 436]                               # the last two continue what the cache holds
    kv, keys, values = filled_cache(nkv, hd, torch.bfloat16, lengths, seed=hd + nh)
    slots = list(range(len(lengths)))
    counts = [n - s for n, s in zip(lengths, starts)]
    batch = described(slots, counts, starts)
    tokens = sum(counts)
    qkv = rand(tokens, (nh + 2 * nkv) * hd, dtype=torch.bfloat16, seed=5)
    out = torch.full((tokens, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
    want = expected_attention(qkv, batch.slots.tolist(), batch.positions.tolist(), keys, values, nh, nkv, hd)
    assert torch.isfinite(out).all()
    assert rel(out.cpu(), want) < 1e-2


def test_matrix_core_attention_finds_a_far_key(ops):
    nh, nkv, hd = 8, 2, 128
    kv, keys, values = filled_cache(nkv, hd, torch.bfloat16, [900], seed=1)
    for far in (0, 5, 63, 64, 500, 899):
        q_row = torch.zeros((nh + 2 * nkv) * hd, dtype=torch.bfloat16, device=DEV)
        for head in range(nh):
            q_row[head * hd:(head + 1) * hd] = keys[0][far, head // 4] * 40.0
        for batch, rows in ((described([0], [1], [899]), 1), (described([0], [40], [860]), 40)):
            qkv = q_row[None, :].repeat(rows, 1).contiguous()
            out = torch.empty(rows, nh * hd, dtype=torch.bfloat16, device=DEV)
            ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
            for head in range(nh):
                got = out[-1, head * hd:(head + 1) * hd].float()
                assert rel(got, values[0][far, head // 4].float()) < 2e-2, (far, head, rows)


# ---- sampling ------------------------------------------------------------------------------

def sample(ops, logits, temperature=0.0, top_k=0, top_p=1.0, penalty=1.0, history=(), draws=None):
    rows = logits.shape[0]
    f = lambda v: torch.full((rows,), float(v), device=DEV)
    offsets = i32([len(history) * (r + e) for r in range(rows) for e in (0, 1)])   # a span (begin, end) per row
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    uniforms = torch.tensor(draws if draws is not None else [0.5] * rows, dtype=torch.float32, device=DEV)
    operands = (logits, out, f(temperature), torch.full((rows,), top_k, dtype=torch.int32, device=DEV), f(top_p),
                f(penalty), i32(list(history) * rows), offsets, uniforms)
    ops.sample(*operands)
    picked = out.tolist()
    # the way through slices (taken by rows with a small top-k, where the vocabulary is large enough) picks the same
    out.fill_(-1)
    ops.sample(*operands, small_top_k=True)
    if temperature > 1e-5 and top_k == 0 and top_p >= 1.0:
        # A draw from all tokens adds up a hundred thousand float32 weights, slice by slice on the one way and run by
        # run on the other: a drawn number that falls on the edge between two tokens may go to either. (What both
        # ways pick is held against float64 sums in test_sample_with_a_temperature_alone_through_slices.)
        other = out.tolist()
        apart = [(a, b) for a, b in zip(picked, other) if a != b]
        assert len(apart) <= max(1, rows // 100) and all(abs(a - b) == 1 for a, b in apart), apart
    else:
        assert out.tolist() == picked
    return picked


def test_sample_reference_cases(ops):
    # tests/sampler_test.rs:101-127 of the reference
    assert sample(ops, torch.tensor([[-1.0, 0.5, 3.25, 2.0]], device=DEV), top_k=1, top_p=0.1) == [2]
    assert sample(ops, torch.tensor([[1.2, 1.5]], device=DEV), penalty=2.0, history=[1]) == [0]
    assert sample(ops, torch.tensor([[1.2, 1.5]], device=DEV), penalty=1.0, history=[1]) == [1]
    assert sample(ops, torch.tensor([[1.0, 3.0, 3.0, float("nan")]], device=DEV)) == [1]   # ties: lowest id; NaN never wins
    # tests/sampler_test.rs:24-98: a draw between p0 and p0+p1 picks token 1 when hot, token 0 when cold
    e = math.exp
    logits = torch.tensor([[2.0, 1.0, 0.0]], device=DEV)
    hot0, hot1 = e(1) / (e(1) + e(0.5) + 1), e(0.5) / (e(1) + e(0.5) + 1)
    draw = hot0 + hot1 / 2
    assert sample(ops, logits, temperature=2.0, draws=[draw]) == [1]
    assert sample(ops, logits, temperature=0.5, draws=[draw]) == [0]
    logits = torch.tensor([[4.0, 3.0, 2.0, 1.0]], device=DEV)
    total = e(4) + e(3) + e(2) + e(1)
    draw = (e(4) + e(3) + e(2) / 2) / total                         # falls on token 2 of the full distribution
    assert sample(ops, logits, temperature=1.0, draws=[draw]) == [2]
    assert sample(ops, logits, temperature=1.0, top_k=2, draws=[draw]) == [1]
    assert sample(ops, logits, temperature=1.0, top_p=0.85, draws=[draw]) == [1]


def distribution_by_sorting(logits, temperature, top_k, top_p):
    """P.sampling_distribution with library sorting instead of a loop over the vocabulary, for large ones
    (the test below holds it against the loop where that is affordable)."""
    vocab = logits.numel()
    order = torch.argsort(-logits.double(), stable=True)[:top_k if top_k > 0 else vocab]       # ties: the lower id first
    kept = logits.double()[order]
    probs = torch.exp((kept - kept[0]) / temperature)
    probs = probs / probs.sum()
    if top_p < 1.0:
        reached = torch.nonzero(torch.cumsum(probs, 0) >= top_p)
        keep = int(reached[0]) + 1 if reached.numel() else probs.numel()
        order, probs = order[:keep], probs[:keep] / probs[:keep].sum()
    dist = torch.zeros(vocab, dtype=torch.float64)
    dist[order] = probs
    return dist


@pytest.mark.parametrize("vocab", [384, 1000, 128256, 300001, (1 << 19) - 7])      # the last two: beyond what goes through slices
def test_sample_matches_the_plain_distribution(ops, vocab):
    g = torch.Generator().manual_seed(vocab)
    row = torch.randn(vocab, generator=g) * 2.0
    history = [3, 7, 7, vocab - 1]
    for temperature, top_k, top_p, penalty in [(1.0, 0, 1.0, 1.0), (0.7, 40, 0.95, 1.1), (1.5, 5, 1.0, 2.0),
                                               (1.0, 0, 0.5, 1.0)]:
        adjusted = P.apply_repetition_penalty(row, history, penalty)
        dist = distribution_by_sorting(adjusted, temperature, top_k, top_p)
        if vocab <= 1000:
            assert float((dist - P.sampling_distribution(adjusted, temperature, top_k, top_p)).abs().max()) < 1e-12
        draws = 512 if vocab < 200000 else 128
        logits = row.to(DEV)[None, :].expand(draws, vocab).contiguous()
        u = ((torch.arange(draws) + 0.5) / draws).tolist()          # an even sweep of the unit interval
        picks = sample(ops, logits, temperature, top_k, top_p, penalty, history, draws=u)
        counts = torch.bincount(torch.tensor(picks), minlength=vocab).double() / draws
        # an even sweep reproduces every probability to within 1/draws per token
        assert float((counts - dist).abs().max()) <= 1.5 / draws + 1e-6
        assert set(torch.nonzero(counts).flatten().tolist()) <= set(torch.nonzero(dist).flatten().tolist())
        if top_k:
            kept = set(torch.topk(adjusted, top_k).indices.tolist())
            assert set(picks) <= kept
        greedy = sample(ops, logits[:2].contiguous(), 0.0, top_k, top_p, penalty, history)
        assert greedy == [P.greedy(adjusted)] * 2


def test_sample_with_ties_by_the_thousand_and_a_large_top_k(ops):
    """What top-k leaves is kept in a short list on the chip when it fits; ties that do not fit, and a
    top-k of thousands, take the path over the whole row. Either way only kept tokens are drawn, and an
    even sweep of draws meets every kept token in proportion."""
    vocab, draws = 5000, 400
    u = ((torch.arange(draws) + 0.5) / draws).tolist()
    flat = torch.zeros(vocab)
    flat[[17, 4000]] = 1.0                                         # two tokens above 4998 that tie
    for top_k, allowed in ((2, {17, 4000}), (3, set(range(vocab)))):    # the third place is a tie of 4998
        picks = sample(ops, flat.to(DEV)[None, :].expand(draws, vocab).contiguous(), 1.0, top_k, 1.0, draws=u)
        assert set(picks) <= allowed
        if top_k == 2:
            assert abs(picks.count(17) - draws / 2) <= 1 and abs(picks.count(4000) - draws / 2) <= 1
        else:
            assert len(set(picks)) > 300                            # spread over the tie, not stuck on the top two
    g = torch.Generator().manual_seed(5)
    row = torch.randn(vocab, generator=g) * 2.0
    for top_k in (1500, 2500):                                      # fits the list narrowly, or not at all
        dist = P.sampling_distribution(row, 1.0, top_k, 0.9)
        picks = sample(ops, row.to(DEV)[None, :].expand(draws, vocab).contiguous(), 1.0, top_k, 0.9, draws=u)
        counts = torch.bincount(torch.tensor(picks), minlength=vocab).double() / draws
        assert float((counts - dist).abs().max()) <= 1.5 / draws + 1e-6
        assert set(torch.nonzero(counts).flatten().tolist()) <= set(torch.nonzero(dist).flatten().tolist())


def test_sample_largest_logit_slice_by_slice(ops):
    """Rows that take the largest logit, in a vocabulary large enough for the way through slices: the first
    index among equals, also when they lie in different slices; NaN never wins; a row of nothing but NaN
    or -inf gives index 0; the penalty counts. (The helper checks both ways against each other.)"""
    vocab = 50000
    torch.manual_seed(11)
    logits = torch.randn(7, vocab)
    logits[0, [40000, 123, 4096 * 5 + 7]] = 9.0                    # equal maxima in three slices: the first index
    logits[1, ::3] = float("nan"); logits[1, 30001] = 8.0          # NaN all over
    logits[2] = float("nan")
    logits[3] = float("-inf")
    logits[4, 49999] = 20.0                                        # the very last token, in the last, partly filled slice
    logits[5, 7] = 5.0; logits[5, 20000] = 4.9                     # the penalty takes the first one down
    logits[6] = -logits[6].abs() - 1.0; logits[6, 33333] = -0.5    # all negative
    logits = logits.to(DEV)
    picked = sample(ops, logits)
    assert picked[:5] == [123, 30001, 0, 0, 49999] and picked[6] == 33333
    assert picked[5] == 7
    assert sample(ops, logits, penalty=1.5, history=[7, 8, 9])[5] == 20000


def test_sample_keeps_the_tokens_on_the_device_where_asked(ops):
    """With append_at the chosen token is also written behind the row's span of the history, on every way
    through the kernels (greedy, passes over the row, candidates from slices), and only for the rows
    that ask for it; what it wrote is what the penalty of the next call reads."""
    torch.manual_seed(5)
    rows, vocab = 5, 40000
    logits = (torch.randn(rows, vocab) * 3.0).to(DEV)
    temperature = torch.tensor([0.0, 0.9, 0.9, 1.0, 0.0], device=DEV)
    top_k = i32([0, 40, 0, 8, 0])
    top_p = torch.tensor([1.0, 0.95, 1.0, 0.9, 1.0], device=DEV)
    penalty = torch.tensor([1.0, 1.2, 1.0, 1.0, 1.0e9], device=DEV)
    uniforms = torch.tensor([0.1, 0.5, 0.7, 0.3, 0.2], device=DEV)
    room = 6
    for small in (False, True):
        history = torch.full((rows * room,), -7, dtype=torch.int32, device=DEV)
        lengths = [0] * rows
        picked = []
        for step in range(3):
            spans = i32([r * room + e * lengths[r] for r in range(rows) for e in (0, 1)])
            append_at = i32([r * room + lengths[r] if r != 2 else -1 for r in range(rows)])   # row 2 keeps nothing
            out = torch.empty(rows, dtype=torch.int32, device=DEV)
            ops.sample(logits, out, temperature, top_k, top_p, penalty, history, spans, uniforms,
                       small_top_k=small, append_at=append_at)
            picked.append(out.tolist())
            lengths = [n + (1 if r != 2 else 0) for r, n in enumerate(lengths)]
        kept = history.view(rows, room).tolist()
        for r in range(rows):
            want = [step[r] for step in picked] if r != 2 else []
            assert kept[r] == want + [-7] * (room - len(want)), (small, r)
        # row 4 is greedy with a crushing penalty: it reads what it wrote and never takes a token twice
        assert len(set(kept[4][:3])) == 3 and picked[0][4] == int(logits[4].argmax())
        assert picked[0][0] == picked[1][0] == int(logits[0].argmax())      # no penalty: the same token again


@pytest.mark.parametrize("vocab", [32768 - 4095, 40000, 151936])
def test_sample_small_top_k_through_slices(ops, vocab):
    """Rows of every kind in one call (greedy, no top-k, top-k of 1, 40 and 64, a penalty, ties that overflow a
    slice's list, ties across slices): the way through slices picks what the passes over the row pick."""
    g = torch.Generator().manual_seed(vocab)
    rows = 12
    logits = torch.randn(rows, vocab, generator=g) * 3.0
    logits[9, torch.randperm(vocab, generator=g)[:12]] += 25.0     # a dozen tokens hold nearly all the mass, as a model's do
    logits[10, torch.randperm(vocab, generator=g)[:70]] += 25.0    # seventy: more than the candidates of a top-p alone
    logits[11, 1000:1100] = 30.0                                   # a hundred that tie at the top
    logits[5, 5000:5300] = 40.0                                    # 300 tokens tie at the top of one slice
    logits[6, ::4096] = 35.0                                       # one token at the top of every slice: they tie across slices
    logits[7] = logits[7].abs() * -1.0                             # all negative
    logits[8, vocab - 3:] = 50.0                                   # the last, partly filled slice holds the largest
    logits = logits.to(DEV)
    temperature = torch.tensor([0.0, 1.0, 0.8, 0.8, 1.3, 1.0, 1.0, 0.7, 1.0, 1.0, 0.9, 1.0], device=DEV)
    top_k = i32([40, 0, 1, 40, 64, 20, 5, 40, 2, 0, 0, 0])         # rows 1 and 9 to 11: a top-p alone
    top_p = torch.tensor([1.0, 0.9, 1.0, 0.95, 0.5, 1.0, 1.0, 0.9, 1.0, 0.9, 0.95, 0.8], device=DEV)
    penalty = torch.tensor([1.0, 1.0, 1.0, 1.1, 2.0, 1.0, 1.0, 1.5, 1.0, 1.0, 1.0, 1.0], device=DEV)
    history = i32(list(range(0, vocab, 997)))
    offsets = i32([0, 0] * 3 + [0, len(history)] + [0, 0] * 8)     # the history is row 3's alone
    for draw in (0.03, 0.37, 0.71, 0.93, 0.999):
        uniforms = torch.full((rows,), draw, device=DEV)
        whole, sliced = torch.empty(rows, dtype=torch.int32, device=DEV), torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        ops.sample(logits, whole, temperature, top_k, top_p, penalty, history, offsets, uniforms)
        ops.sample(logits, sliced, temperature, top_k, top_p, penalty, history, offsets, uniforms, small_top_k=True)
        assert sliced.tolist() == whole.tolist()
    picks = whole.tolist()
    assert picks[2] == int(logits[2].argmax())                     # top-k 1
    assert 5000 <= picks[5] < 5300 and picks[6] % 4096 == 0 and picks[8] >= vocab - 3
    assert float(logits[9, picks[9]]) > 15.0 and float(logits[10, picks[10]]) > 15.0 and 1000 <= picks[11] < 1100


@pytest.mark.parametrize("vocab", [32768 - 4095, 128256, 151936])
def test_sample_with_a_temperature_alone_through_slices(ops, vocab):
    """No top-k and no top-p: the inverse CDF over all tokens in the order of ids. The slices' masses say where the drawn
    number falls; the token picked is the one at which the cumulative mass (float64, on the host) passes it."""
    g = torch.Generator().manual_seed(vocab + 1)
    rows = 6
    logits = torch.randn(rows, vocab, generator=g) * 2.0
    logits[1, torch.randperm(vocab, generator=g)[:20]] += 12.0     # a few tokens hold most of the mass
    logits[2, vocab - 5:] += 9.0                                   # much of it in the last, partly filled slice
    logits[3] = logits[3].abs() * -1.0
    logits[5, :4096] = -float("inf")                               # a first slice without mass
    temperature = [1.0, 0.7, 1.5, 0.9, 1.0, 1.0]
    penalty = [1.0, 1.0, 1.0, 1.8, 1.3, 1.0]
    history = list(range(3, vocab, 389))                           # rows 3 and 4 have seen these
    offsets = [0, 0] * 3 + [0, len(history)] * 2 + [0, 0]
    adjusted = logits.double().clone()
    for r in (3, 4):
        seen = adjusted[r, history]
        adjusted[r, history] = torch.where(seen > 0, seen / penalty[r], seen * penalty[r])
    weights = torch.exp((adjusted - adjusted.max(dim=1, keepdim=True).values) / torch.tensor(temperature).double()[:, None])
    through = weights.cumsum(dim=1)
    device_logits = logits.to(DEV)
    for draw in (0.0, 0.013, 0.25, 0.5, 0.77, 0.999, 0.9999999):
        out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        ops.sample(device_logits, out, torch.tensor(temperature, device=DEV), i32([0] * rows), torch.ones(rows, device=DEV),
                   torch.tensor(penalty, device=DEV), i32(history), i32(offsets), torch.full((rows,), draw, device=DEV),
                   small_top_k=True)
        whole = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        ops.sample(device_logits, whole, torch.tensor(temperature, device=DEV), i32([0] * rows), torch.ones(rows, device=DEV),
                   torch.tensor(penalty, device=DEV), i32(history), i32(offsets), torch.full((rows,), draw, device=DEV))
        for r, (pick, other) in enumerate(zip(out.tolist(), whole.tolist())):
            for way, token in (("slices", pick), ("passes", other)):
                assert 0 <= token < vocab and float(weights[r, token]) > 0.0, (way, r, draw, token)
                target = draw * float(through[r, -1])
                before = float(through[r, token - 1]) if token > 0 else 0.0
                slack = 2e-5 * float(through[r, -1])               # float32 sums of up to 150 k weights
                assert before <= target + slack and float(through[r, token]) >= target - slack, (way, r, draw, token)


def test_sample_rows_are_independent(ops):
    g = torch.Generator().manual_seed(1)
    logits = (torch.randn(5, 777, generator=g) * 3).to(DEV)
    u = [0.1, 0.5, 0.9, 0.3, 0.7]
    together = sample(ops, logits, 0.9, 50, 0.9, 1.0, draws=u)
    alone = [sample(ops, logits[r:r + 1].contiguous(), 0.9, 50, 0.9, 1.0, draws=[u[r]])[0] for r in range(5)]
    assert together == alone



# ---- every kernel once more, against the plain C++ references -------------------------------------

@pytest.fixture(scope="module")
def cpp():
    from reference_cpp import CppReference
    return CppReference()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_elementwise_and_products_against_the_cpp_references(ops, cpp, dtype):
    table, ids = rand(333, 96, dtype=DT[dtype], seed=1), i32([0, 332, 7, 7])
    out = torch.empty(4, 96, device=DEV)
    ops.embed(table, ids, out)
    assert torch.equal(out.cpu(), cpp.embed(table, ids))
    x, gain = rand(6, 1000, seed=2, scale=3.0), (rand(1000, seed=3) + 1.0).to(DT[dtype])
    normed = torch.empty(6, 1000, dtype=DT[dtype], device=DEV)
    ops.rmsnorm(x, gain, 1e-4, normed)
    assert rel(normed.float().cpu(), cpp.rmsnorm(x, gain, 1e-4)) < ULP[dtype]
    for m, n, k in ((3, 40, 96), (16, 176, 64), (40, 520, 256), (300, 130, 192)):
        a, w = rand(m, k, dtype=DT[dtype], seed=m), rand(2 * n, k, dtype=DT[dtype], seed=n, scale=0.2)
        stored = torch.empty(m, 2 * n, device=DEV)
        ops.linear(a, w, stored)
        assert rel(stored.cpu(), cpp.linear(a, w)) < 2e-5
        base = rand(m, 2 * n, seed=9)
        summed = base.clone()
        ops.linear(a, w, summed, accumulate=True)
        assert rel(summed.cpu(), cpp.linear(a, w, base=base)) < 2e-5
        gated = torch.empty(m, n, dtype=DT[dtype], device=DEV)
        ops.linear_glu(a, w, gated)
        assert rel(gated.float().cpu(), cpp.linear_glu(a, w)) < ULP[dtype] * 2
        if dtype == "bfloat16" and k % 32 == 0 and n % 8 == 0:          # the same from packed weights; and the packing itself
            ops.linear_glu(a, ops.pack(w, "gated", gated_n=n), gated)
            assert rel(gated.float().cpu(), cpp.linear_glu(a, w)) < ULP[dtype] * 2
            assert torch.equal(ops.pack(w, "gated", gated_n=n).data.float().cpu(), cpp.pack(w, kind=2, gated_n=n))
            assert torch.equal(ops.pack(w, "rotary", head_dim=16, rotated_heads=n // 16).data.float().cpu(),
                               cpp.pack(w, kind=3, head_dim=16, rotated_heads=n // 16))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd", [(4, 2, 32), (8, 2, 128), (6, 3, 64)])
def test_preparation_and_attention_against_the_cpp_references(ops, cpp, dtype, nh, nkv, hd):
    """A prompt of 150 tokens, then one token more (the matrix-core kernels in bfloat16 at head sizes 64 and 128,
    the general kernel otherwise): the rows and the cache after the preparation, and the attention's output."""
    width, eps = (nh + 2 * nkv) * hd, 1e-4
    theta = (torch.tensor(10000.0) ** (torch.arange(hd // 2) * 2.0 / hd))
    qn, kn = rand(hd, seed=1).cpu() + 1.0, rand(hd, seed=2).cpu() + 1.0
    kv = make_cache(5, nkv, hd, DT[dtype], 1, 4)
    kv.block_table[0, :3] = i32([4, 1, 2])
    host_k, host_v = torch.zeros(5, nkv, 64, hd), torch.zeros(5, nkv, hd, 64)
    tol = 3e-5 if dtype == "float32" else ULP[dtype]
    for count, start in ((150, 0), (1, 150)):
        batch = described([0], [count], [start])
        qkv = rand(count, width, dtype=DT[dtype], seed=count)
        want = cpp.qkv_prepare(qkv, nh, nkv, hd, batch.positions, batch.slots, qn, kn, eps, theta, hd, 1.0,
                               kv=(host_k, host_v, kv.block_table.cpu()))
        ops.qkv_prepare(qkv, nh, nkv, hd, batch.positions, batch.slots, q_norm=qn.to(DEV), k_norm=kn.to(DEV), norm_eps=eps,
                        rope_theta=theta.to(DEV), rope_dim=hd, kv=kv, longest_run=count)
        assert rel(qkv.float().cpu(), want) < tol
        assert rel(kv.k.float().cpu(), host_k) < tol and rel(kv.v.float().cpu(), host_v) < tol
        out = torch.empty(count, nh * hd, dtype=DT[dtype], device=DEV)
        ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
        # the reference on exactly what the kernel read: the prepared rows and the cache as the device holds them
        expected = cpp.attention(qkv, nh, nkv, hd, kv.k, kv.v, kv.block_table, batch.positions, batch.slots, 1.0 / math.sqrt(hd))
        assert rel(out.float().cpu(), expected) < (2e-5 if dtype == "float32" else 2e-2)


def test_sampling_and_random_weights_against_the_cpp_references(ops, cpp):
    from xeno_rt_amd.weights import random_init
    vocab, rows = 5000, 64
    logits = rand(rows, vocab, seed=5, scale=2.0)
    history = [3, 7, 7, vocab - 1]
    u = ((torch.arange(rows) + 0.5) / rows).tolist()
    for temperature, top_k, top_p, penalty in [(0.0, 0, 1.0, 1.0), (1.0, 0, 1.0, 1.0), (0.7, 40, 0.95, 1.1), (1.5, 5, 1.0, 2.0)]:
        got = sample(ops, logits, temperature, top_k, top_p, penalty, history, draws=u)
        want = cpp.sample(logits, [temperature] * rows, [top_k] * rows, [top_p] * rows, [penalty] * rows,
                          history * rows, [len(history) * (r + e) for r in range(rows) for e in (0, 1)], u)
        # weights are summed in another order: a draw that falls on the edge between two tokens may take the neighbour
        assert sum(a != b for a, b in zip(got, want)) <= 1, (temperature, top_k, top_p, penalty)
    key = random_init.tensor_key(3, "w")
    out = torch.empty(100000, device=DEV)
    ops.random_normal(out, key, random_init.normal_scale(0.02), 0.0)
    assert torch.equal(out.cpu(), cpp.random_normal(100000, key, random_init.normal_scale(0.02)))
