"""Each HIP kernel alone against its plain torch reference (tests/ref_ops.py), at sizes other than the engine's."""
import math

import pytest
import torch

from . import ref_ops
from .tiny import rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"f32": torch.float32, "bf16": torch.bfloat16}


@pytest.fixture(scope="module")
def ops():
    from trapetum_amd import kernels
    return kernels.load(torch.device(DEV))


def randn(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def tol(dtype):
    return 2e-6 if dtype == torch.float32 else 6e-3


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("m,d,v", [(1, 64, 17), (5, 88, 331), (33, 2304, 1000)])
def test_embed_rows(ops, dt, m, d, v):
    table = randn(v, d, dtype=DT[dt])
    tok = torch.randint(0, v, (m,), dtype=torch.int32, device=DEV)
    got = ops.embed_rows(tok, table, math.sqrt(d))
    assert torch.equal(got.cpu(), ref_ops.embed_rows(tok.cpu(), table.cpu(), math.sqrt(d)))


@pytest.mark.parametrize("din,dout", [("f32", "f32"), ("f32", "bf16"), ("bf16", "bf16"), ("bf16", "f32")])
@pytest.mark.parametrize("m,d", [(1, 16), (3, 88), (7, 2304), (2, 5000)])
def test_rms_norm(ops, din, dout, m, d):
    x = randn(m, d, dtype=DT[din], seed=1, scale=3.0)
    gain = 1.0 + randn(d, seed=2, scale=0.3)
    got = ops.rms_norm(x, gain, 1e-5, DT[dout])
    ref = ref_ops.rms_norm(x.cpu(), gain.cpu(), 1e-5, DT[dout])
    assert rel_l2(got, ref) < tol(DT[dout])


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("post,nxt", [(True, True), (True, False), (False, True), (False, False)])
@pytest.mark.parametrize("m,d", [(1, 64), (5, 88), (4, 3584),
                                 # many rows: four elements per lane, one width for each of its forms and their edges
                                 (130, 88), (200, 1000), (150, 2304), (140, 3072), (129, 4608), (130, 8192), (131, 8200), (130, 90),
                                 # few rows of many chunks: a chunk a lane, every form and its edges
                                 (8, 1028), (3, 2304), (64, 2560), (5, 2564), (2, 4096), (7, 4608), (9, 5120), (4, 5124), (6, 8192)])
def test_add_rms_norm(ops, dt, post, nxt, m, d):
    stream = randn(m, d, seed=3, scale=2.0)
    rows = randn(m, d, dtype=DT[dt], seed=4, scale=5.0)
    gp = (1.0 + randn(d, seed=5, scale=0.2)) if post else None
    gn = (1.0 + randn(d, seed=6, scale=0.2)) if nxt else None
    ref_stream = stream.cpu().clone()
    ref = ref_ops.add_rms_norm(ref_stream, rows.cpu(), gp.cpu() if post else None, 1e-6, gn.cpu() if nxt else None, 1e-4, DT[dt])
    got = ops.add_rms_norm(stream, rows, gp, 1e-6, gn, 1e-4, DT[dt])
    assert rel_l2(stream, ref_stream) < 2e-6
    if nxt:
        assert rel_l2(got, ref) < tol(DT[dt])
    else:
        assert got is None


@pytest.mark.parametrize("m,n,k", [(8, 2304, 2048), (3, 600, 9216), (64, 2304, 4096), (700, 2304, 2048), (300, 520, 4104),
                                   (2048, 2304, 4096), (1, 2304, 9216), (2, 601, 14336),
                                   (5, 2304, 9216), (8, 77, 1544), (4, 4608, 4096), (7, 1000, 20000)])
def test_deferred_product_into_add_rms_norm(ops, m, n, k):
    """A product left in K slices and added by add_rms_norm equals the product, then the norm."""
    from trapetum_amd.kernels.ops import SplitRows
    x, w = randn(m, k, dtype=torch.bfloat16, seed=70), randn(n, k, dtype=torch.bfloat16, seed=71, scale=0.05)
    rows = ops.linear(x, w, torch.bfloat16, defer=True)
    assert isinstance(rows, SplitRows) and rows.shape == (m, n) and rows.slices.shape[0] > 1
    ref_rows = x.cpu().double() @ w.cpu().double().T
    assert rel_l2(ops.rows(rows, torch.float32), ref_rows) < 1e-5
    stream = randn(m, n, seed=72)
    gp, gn = 1.0 + randn(n, seed=73, scale=0.2), 1.0 + randn(n, seed=74, scale=0.2)
    ref_stream = stream.cpu().clone()
    ref = ref_ops.add_rms_norm(ref_stream, ref_rows.float(), gp.cpu(), 1e-6, gn.cpu(), 1e-6, torch.float32)
    got = ops.add_rms_norm(stream, rows, gp, 1e-6, gn, 1e-6, torch.bfloat16)
    assert rel_l2(stream, ref_stream) < 1e-5 and rel_l2(got, ref) < 6e-3


def test_rows_wider_than_the_fused_kernel_takes_are_added_first(ops):
    """A product in K slices whose rows are wider than `add_rms_norm` keeps in registers (8192): the slices are added by
    a kernel of their own, in slice order, and the result is what the fused path gives for narrower rows."""
    m, d = 5, 8192 + 8
    slices = randn(3, m, d, seed=70)
    stream = randn(m, d, seed=71)
    gp, gn = randn(d, seed=72).abs() + 0.5, randn(d, seed=73).abs() + 0.5
    ref_stream = stream.cpu().clone()
    ref = ref_ops.add_rms_norm(ref_stream, slices.cpu().sum(0), gp.cpu(), 1e-5, gn.cpu(), 1e-6, torch.bfloat16)
    from trapetum_amd.kernels.ops import SplitRows
    got = ops.add_rms_norm(stream, SplitRows(slices), gp, 1e-5, gn, 1e-6, torch.bfloat16)
    assert rel_l2(stream, ref_stream) < 3e-3 and rel_l2(got, ref) < 6e-3
    summed = ops.rows(SplitRows(slices), torch.float32)
    assert torch.equal(summed.cpu(), (slices[0] + slices[1] + slices[2]).cpu())
    # a product may leave its slices to the consumer only without an epilogue
    x, w = randn(8, 64, dtype=torch.bfloat16, seed=74), randn(128, 64, dtype=torch.bfloat16, seed=75)
    y = torch.empty(8, 128, dtype=torch.float32, device=DEV)
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=DEV)
    rc = ops.lib.tp_linear(x.data_ptr(), w.data_ptr(), y.data_ptr(), 1, 0, 8, 128, 64, 1, 30.0, 0, 0, ws.data_ptr(), 1 << 20, 1, 0, None)
    assert rc != 0 and b"epilogue" in ops.lib.tp_last_error()


def test_gather_rows(ops):
    x = randn(9, 88)
    rows = torch.tensor([8, 0, 3, 3], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.gather_rows(x, rows).cpu(), x.cpu()[[8, 0, 3, 3]])


# ---- matrix products: every kernel, ragged edges -------------------------------------------------------
LINEAR_SHAPES = [(1, 16, 8), (3, 100, 72), (17, 331, 88), (64, 130, 2304), (5, 2304, 2048), (8, 1000, 9216),
                 (65, 200, 136), (300, 257, 520)]


LINEAR_SHAPES += [(65, 100, 64), (300, 257, 576), (1000, 520, 192), (513, 2304, 2048)]
# grids of more than a thousand tiles, which the tiled kernel walks in another order (per XCD, in panels): tile counts
# that are no multiple of 8 and a last panel that is not whole
LINEAR_SHAPES += [(300, 44177, 64), (40, 70001, 72)]


# one and two rows, for the kernel that takes no more: widths of one to ten chunks a lane, an odd number of rows of W
LINEAR_SHAPES += [(1, 77, 8), (2, 301, 1000), (2, 130, 1536), (1, 257, 3584), (2, 99, 4608), (1, 64, 5120)]


# three to eight rows, for the kernel of blocks of 8 rows of W: an N that is no multiple of 8 or 16, a K that ends inside a
# step of 64, inside a wave's quarter and in a second round of loads, every number of rows of X
LINEAR_SHAPES += [(3, 77, 8), (8, 1001, 2304), (7, 130, 2312), (6, 250, 5000), (4, 4099, 600), (5, 9, 9216)]


# nine to 64 rows: every number of 16-row groups of X, an N and a K that end inside a tile and inside a k step, K slices
# whose number a whole number of k steps makes smaller than was asked for
LINEAR_SHAPES += [(9, 77, 64), (33, 1001, 2304), (48, 130, 2312), (64, 250, 5000), (20, 4099, 600), (50, 9, 9216), (16, 64, 72)]


@pytest.mark.parametrize("algo", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11])
@pytest.mark.parametrize("m,n,k", LINEAR_SHAPES)
def test_linear_bf16(ops, algo, m, n, k):
    if algo in (8, 9) and k % 64:
        pytest.skip("the loop that loads straight into LDS takes whole k steps of 64")
    if algo == 2 and m > 64:
        pytest.skip("the skinny kernel takes at most 64 rows")
    if algo == 4 and (m > 2 or k > 5120):
        pytest.skip("the multiply-add kernel takes at most 2 rows and, unsliced, a K of 5120")
    if algo == 5 and m > 8:
        pytest.skip("the kernel of 8-row blocks takes at most 8 rows")
    x, w = randn(m, k, dtype=torch.bfloat16, seed=7), randn(n, k, dtype=torch.bfloat16, seed=8, scale=0.05)
    ops.force_linear = algo
    try:
        got_b = ops.linear(x, w, torch.bfloat16)
        got_f = ops.linear(x, w, torch.float32)
        got_c = ops.linear(x, w, torch.float32, softcap=3.0)
        got_d = ops.rows(ops.linear(x, w, torch.bfloat16, defer=True), torch.float32)      # K slices, where the kernel makes them
    finally:
        ops.force_linear = 0
    ref = x.cpu().double() @ w.cpu().double().T
    assert rel_l2(got_f, ref) < 1e-5
    assert rel_l2(got_b, ref) < 4e-3
    assert rel_l2(got_c, 3.0 * torch.tanh(ref / 3.0)) < 1e-5
    assert rel_l2(got_d, ref) < 4e-3


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("m,n,k", [(1, 16, 8), (8, 2304, 2048), (70, 331, 88), (300, 77, 136)])
def test_linear_with_a_bias(ops, dt, m, n, k):
    """x @ w^T + bias, the bias added by a kernel of its own after whichever product kernel the shape takes."""
    x, w = randn(m, k, dtype=DT[dt], seed=17), randn(n, k, dtype=DT[dt], seed=18, scale=0.05)
    bias = randn(n, seed=19)
    got = ops.linear(x, w, DT[dt], bias=bias)
    ref = x.cpu().double() @ w.cpu().double().T + bias.cpu().double()
    assert got.shape == (m, n) and rel_l2(got, ref) < (2e-6 if dt == "f32" else 4e-3)
    assert rel_l2(ops.linear(x, w, DT[dt], defer=True, bias=bias), ref) < (2e-6 if dt == "f32" else 4e-3)   # never left in slices
    with pytest.raises(Exception, match="bias"):
        ops.linear(x, w, DT[dt], softcap=30.0, bias=bias)
    with pytest.raises(Exception, match="bias"):
        ops.linear(x, w, DT[dt], bias=bias[:-1].contiguous())


@pytest.mark.parametrize("m,n,k", [(1, 16, 8), (3, 100, 71), (70, 331, 88), (5, 700, 2304)])
def test_linear_f32(ops, m, n, k):
    x, w = randn(m, k, seed=9), randn(n, k, seed=10, scale=0.05)
    got = ops.linear(x, w, torch.float32)
    ref = x.cpu().double() @ w.cpu().double().T
    assert rel_l2(got, ref) < 2e-6
    # the sum's order per element does not depend on the other rows: a row alone gives the same bits
    alone = ops.linear(x[m - 1:m].contiguous(), w, torch.float32)
    assert torch.equal(alone[0], got[m - 1])


@pytest.mark.parametrize("algo", [1, 2, 3, 4, 5, 6, 8, 10, 11])
@pytest.mark.parametrize("dt", ["bf16", "f32"])
@pytest.mark.parametrize("m,inter,k", [(1, 16, 16), (4, 200, 88), (40, 320, 96), (9, 1000, 2304), (150, 72, 136),
                                       (150, 72, 128), (700, 1000, 320), (130, 36010, 64), (2, 1000, 2304), (1, 75, 4608),
                                       (8, 9216, 2304), (3, 41, 2504), (7, 8, 520), (64, 9216, 2304), (33, 1000, 200),
                                       (17, 41, 2504), (48, 8, 520)])
def test_gated_linear(ops, algo, dt, m, inter, k):
    if dt == "f32" and algo != 1:
        pytest.skip("float32 runs on the plain kernel only")
    if algo == 4 and m > 2:
        pytest.skip("the multiply-add kernel takes at most 2 rows")
    if algo == 5 and m > 8:
        pytest.skip("the kernel of 8-row blocks takes at most 8 rows")
    if algo == 2 and m > 64:
        pytest.skip("the skinny kernel takes at most 64 rows")
    if algo in (8, 9) and k % 64:
        pytest.skip("the loop that loads straight into LDS takes whole k steps of 64")
    wg, wu = randn(inter, k, dtype=DT[dt], seed=11, scale=0.2), randn(inter, k, dtype=DT[dt], seed=12, scale=0.2)
    x = randn(m, k, dtype=DT[dt], seed=13)
    packed = ops.pack_gate_up(wg, wu)
    assert torch.equal(packed.cpu(), ref_ops.pack_gate_up(wg.cpu(), wu.cpu()))
    ops.force_linear = algo
    try:
        got = ops.gated_linear(x, packed, inter, "gelu_tanh", DT[dt])
        silu = ops.gated_linear(x, packed, inter, "silu", DT[dt])
        with pytest.raises(Exception, match="no kernel"):
            ops.gated_linear(x, packed, inter, "relu", DT[dt])
    finally:
        ops.force_linear = 0
    g, u = x.cpu().double() @ wg.cpu().double().T, x.cpu().double() @ wu.cpu().double().T
    ref = torch.nn.functional.gelu(g, approximate="tanh") * u
    assert rel_l2(got, ref) < (5e-6 if dt == "f32" else 4e-3)
    assert rel_l2(silu, torch.nn.functional.silu(g) * u) < (5e-6 if dt == "f32" else 4e-3)      # the other activation offered


@pytest.mark.parametrize("algo,m", [(2, 8), (3, 8), (3, 200), (5, 8), (5, 3)])
def test_gated_linear_at_the_ends_of_the_activation(ops, algo, m):
    """Gate values far out on both sides (the activation is the identity on one, zero on the other): no overflow of the
    exponential shows in the result."""
    k, inter = 64, 96
    wg, wu = randn(inter, k, dtype=torch.bfloat16, seed=14), randn(inter, k, dtype=torch.bfloat16, seed=15, scale=0.2)
    x = randn(m, k, dtype=torch.bfloat16, seed=16)
    x[::2] *= 1.0e4
    x[1::4] *= 1.0e15
    ops.force_linear = algo
    try:
        got = ops.gated_linear(x, ops.pack_gate_up(wg, wu), inter, "gelu_tanh", torch.float32)
    finally:
        ops.force_linear = 0
    g, u = x.cpu().double() @ wg.cpu().double().T, x.cpu().double() @ wu.cpu().double().T
    ref = torch.nn.functional.gelu(g, approximate="tanh") * u
    assert torch.isfinite(got).all()
    assert rel_l2(got, ref) < 1e-5


# ---- RoPE + cache write, attention over pages --------------------------------------------------------------
def build_cache_case(dt, H, KV, hd, lens, page, rows_cap, n_pages, seed):
    """Random q/k/v rows for sequences of the given lengths, pushed through rope_kv_write of the reference."""
    m = sum(lens)
    q = randn(m, H * hd, dtype=dt, seed=seed)
    k = randn(m, KV * hd, dtype=dt, seed=seed + 1)
    v = randn(m, KV * hd, dtype=dt, seed=seed + 2)
    row_seq = torch.repeat_interleave(torch.arange(len(lens)), torch.tensor(lens)).to(torch.int32)
    row_pos = torch.cat([torch.arange(n) for n in lens]).to(torch.int32)
    new_len = torch.tensor(lens, dtype=torch.int32)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed)).tolist()
    width = max(-(-(min(n, rows_cap) if rows_cap else n) // page) for n in lens)
    table = torch.full((len(lens), width), -1, dtype=torch.int32)
    for i, n in enumerate(lens):
        need = -(-(min(n, rows_cap) if rows_cap else n) // page)
        for j in range(need):
            table[i, j] = perm.pop()
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd)))
    return dict(q=q, k=k, v=v, row_seq=row_seq, row_pos=row_pos, new_len=new_len, cu=cu, table=table, inv_freq=inv_freq)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("H,KV,hd,lens,page,rows_cap", [
    (4, 2, 16, (5, 11, 17), 16, 0), (6, 1, 32, (1, 9, 23, 40), 16, 16), (3, 3, 48, (70, 3), 64, 64),
    (8, 4, 256, (130,), 64, 0), (2, 2, 80, (33, 50), 16, 32), (4, 2, 64, (200, 90), 16, 0), (5, 1, 32, (300,), 16, 64),
    (2, 2, 80, (150, 140), 16, 0), (8, 4, 256, (300, 77), 64, 128)])
def test_rope_kv_write(ops, dt, H, KV, hd, lens, page, rows_cap):
    c = build_cache_case(DT[dt], H, KV, hd, lens, page, rows_cap, 24, 20)
    rot = hd if hd != 80 else 48                            # one head size with a rotation over part of the head
    c["inv_freq"] = c["inv_freq"][:rot // 2].contiguous()
    pools_ref = [torch.zeros(24, KV, page, hd, dtype=DT[dt]) for _ in range(2)]
    pools = [p.to(DEV) for p in pools_ref]
    q_ref, k_ref = c["q"].cpu().clone(), c["k"].cpu().clone()
    ref_ops.rope_kv_write(q_ref, k_ref, c["v"].cpu(), H, KV, hd, c["inv_freq"], rot, c["row_seq"], c["row_pos"],
                          c["new_len"], c["table"], pools_ref[0], pools_ref[1], rows_cap)
    ops.rope_kv_write(c["q"], c["k"], c["v"], H, KV, hd, c["inv_freq"].to(DEV), rot, c["row_seq"].to(DEV),
                      c["row_pos"].to(DEV), c["new_len"].to(DEV), c["table"].to(DEV), pools[0], pools[1], rows_cap)
    t = 3e-6 if dt == "f32" else 6e-3
    assert rel_l2(c["q"], q_ref) < t and rel_l2(c["k"], k_ref) < t
    assert rel_l2(pools[0], pools_ref[0]) < t
    assert torch.equal(pools[1].cpu(), pools_ref[1])
    # rows that no sequence owns stay untouched
    assert torch.equal((pools[0].cpu() != 0).any(dim=-1), (pools_ref[0] != 0).any(dim=-1))


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("H,KV,hd,lens,page,rows_cap,rot", [
    (4, 2, 16, (5, 11, 17), 16, 0, 16), (2, 2, 80, (33, 50), 16, 32, 48), (8, 4, 256, (300, 77), 64, 128, 256),
    (3, 1, 64, (290,), 16, 0, 32)])
def test_rope_kv_write_turning_neighbours(ops, dt, H, KV, hd, lens, page, rows_cap, rot):
    """The other pairing: elements 2d and 2d + 1 turn together by the angle of pair d; few rows and many, a rotation over
    part of the head, a ring."""
    c = build_cache_case(DT[dt], H, KV, hd, lens, page, rows_cap, 24, 21)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot)))
    pools_ref = [torch.zeros(24, KV, page, hd, dtype=DT[dt]) for _ in range(2)]
    pools = [p.to(DEV) for p in pools_ref]
    q_ref, k_ref = c["q"].cpu().clone(), c["k"].cpu().clone()
    halves = c["q"].cpu().clone()
    ref_ops.rope_kv_write(q_ref, k_ref, c["v"].cpu(), H, KV, hd, inv_freq, rot, c["row_seq"], c["row_pos"],
                          c["new_len"], c["table"], pools_ref[0], pools_ref[1], rows_cap, pairing="neighbours")
    ref_ops.rope_kv_write(halves, None, None, H, KV, hd, inv_freq, rot, c["row_seq"], c["row_pos"], c["new_len"], c["table"],
                          None, None, rows_cap)
    assert rel_l2(halves, q_ref) > 0.1                       # the two pairings are not the same rotation
    ops.rope_kv_write(c["q"], c["k"], c["v"], H, KV, hd, inv_freq.to(DEV), rot, c["row_seq"].to(DEV),
                      c["row_pos"].to(DEV), c["new_len"].to(DEV), c["table"].to(DEV), pools[0], pools[1], rows_cap,
                      pairing="neighbours")
    t = 3e-6 if dt == "f32" else 6e-3
    assert rel_l2(c["q"], q_ref) < t and rel_l2(c["k"], k_ref) < t
    assert rel_l2(pools[0], pools_ref[0]) < t
    assert torch.equal(pools[1].cpu(), pools_ref[1])
    with pytest.raises(Exception, match="pairing"):
        ops.rope_kv_write(c["q"], c["k"], c["v"], H, KV, hd, inv_freq.to(DEV), rot, c["row_seq"].to(DEV),
                          c["row_pos"].to(DEV), c["new_len"].to(DEV), c["table"].to(DEV), pools[0], pools[1], rows_cap,
                          pairing="thirds")


ATTN_CASES = [
    # H, KV, hd, lens, page, window, rows_cap, cap
    (4, 2, 16, (5, 11, 17), 16, 8, 16, 50.0),
    (6, 1, 32, (1, 9, 23, 40), 16, 16, 16, 20.0),
    (3, 3, 48, (70, 3), 16, 5, 16, 8.0),
    (8, 4, 256, (130, 64), 64, 0, 0, 50.0),
    (8, 4, 256, (200,), 64, 100, 128, 0.0),
    (2, 2, 80, (33, 50), 16, 0, 0, 0.0),
    (16, 2, 128, (300, 17, 129), 64, 0, 0, 30.0),
    (32, 1, 64, (90,), 16, 0, 0, 0.0),
]


@pytest.mark.parametrize("kernel", ["plain", 0, 1, 2, 3])
@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("H,KV,hd,lens,page,window,rows_cap,cap", ATTN_CASES)
def test_attention_prefill(ops, kernel, dt, H, KV, hd, lens, page, window, rows_cap, cap):
    """kernel: the plain one, or the matrix-core kernel with its block shape (0: its own choice)."""
    plain = kernel == "plain"
    if dt == "f32" and not plain:
        pytest.skip("float32 runs on the plain kernel only")
    c = build_cache_case(DT[dt], H, KV, hd, lens, page, rows_cap, 24, 30)
    scale = 1.0 / math.sqrt(hd * 0.7)
    ref = ref_ops.attention_prefill(c["q"].cpu(), c["k"].cpu(), c["v"].cpu(), H, KV, hd, c["cu"], max(lens), scale,
                                    cap, window, torch.float32)
    ops.force_plain_attention = plain
    try:
        got = ops.attention_prefill(c["q"], c["k"], c["v"], H, KV, hd, c["cu"].to(DEV), max(lens), scale, cap, window,
                                    DT[dt], row_seq=c["row_seq"].to(DEV), row_pos=c["row_pos"].to(DEV),
                                    shape=0 if plain else kernel)
    finally:
        ops.force_plain_attention = False
    assert rel_l2(got, ref) < (3e-6 if dt == "f32" else 8e-3)


@pytest.mark.parametrize("shape", [0, 1, 2, 3])
@pytest.mark.parametrize("H,KV,hd,lens,window,cap", [(64, 8, 16, (450, 130, 64), 100, 30.0), (8, 4, 256, (3300,), 0, 50.0),
                                                    (8, 4, 256, (1000, 77), 300, 0.0), (12, 4, 128, (700, 1), 0, 30.0),
                                                    (6, 2, 80, (333,), 64, 0.0), (4, 4, 48, (97, 300), 0, 20.0)])
def test_attention_prefill_many_tiles(ops, shape, H, KV, hd, lens, window, cap):
    """Steps of many and of few query tiles in every block shape of the kernel (column groups that are heads of a kv
    head or further positions; one, two or four groups of keys), against dense masked attention per sequence and
    head."""
    m, g, scale = sum(lens), H // KV, 1.0 / math.sqrt(hd * 0.7)
    q, k, v = (randn(m, n * hd, dtype=torch.bfloat16, seed=40 + i) for i, n in enumerate((H, KV, KV)))
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    ref = torch.zeros(m, H, hd)
    for i, n in enumerate(lens):
        rows = slice(int(cu[i]), int(cu[i + 1]))
        qs, ks, vs = (t.cpu().float()[rows].reshape(n, -1, hd) for t in (q, k, v))
        pos = torch.arange(n)
        hidden = (pos[None, :] > pos[:, None]) | ((pos[:, None] - pos[None, :] >= window) if window else False)
        for h in range(H):
            s = qs[:, h] @ ks[:, h // g].T * scale
            if cap:
                s = cap * torch.tanh(s / cap)
            ref[rows, h] = torch.softmax(s.masked_fill(hidden, float("-inf")), dim=-1) @ vs[:, h // g]
    got = ops.attention_prefill(q, k, v, H, KV, hd, cu.to(DEV), max(lens), scale, cap, window, torch.bfloat16, shape=shape)
    assert rel_l2(got.reshape(m, H, hd), ref) < 8e-3


EXTEND_CASES = [
    # H, KV, hd, lens, starts (what the cache already holds), page, window, rows_cap, cap
    (4, 2, 16, (25, 11, 17), (20, 0, 16), 16, 8, 16, 50.0),
    (6, 1, 32, (50, 9, 23, 40), (17, 8, 0, 1), 16, 16, 16, 20.0),         # a ring without a row to spare
    (3, 3, 48, (70, 3), (64, 2), 16, 5, 16, 8.0),
    (8, 4, 256, (330, 64), (130, 63), 64, 0, 0, 50.0),
    (8, 4, 256, (700,), (451,), 64, 128, 128, 0.0),                       # the portion is longer than the ring
    (2, 2, 80, (33, 50), (0, 31), 16, 0, 0, 0.0),
    (16, 2, 128, (1300, 17, 129), (1234, 0, 128), 64, 512, 512, 30.0),
    (32, 1, 64, (90,), (89,), 16, 0, 0, 0.0),
    # portions of hundreds of rows, which the rotation and cache write take 16 bytes at a time
    (8, 4, 256, (700, 300), (300, 20), 64, 0, 0, 50.0),
    (4, 2, 64, (600,), (200,), 16, 128, 128, 30.0),
]


@pytest.mark.parametrize("kernel", ["plain", 0, 1, 2, 3])
@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("H,KV,hd,lens,starts,page,window,rows_cap,cap", EXTEND_CASES)
def test_attention_over_cached_positions_and_the_steps_rows(ops, kernel, dt, H, KV, hd, lens, starts, page, window, rows_cap, cap):
    """A step that continues sequences by several tokens: the queries attend over the cached positions, read in place
    through the page table (a ring's rows too), and over the step's own rows, which are cached only afterwards.
    Against whole-sequence attention of the reference; afterwards the cache holds what a whole-sequence step would
    have left.  kernel: the plain one, or the matrix-core kernel with its block shape (0: its own choice)."""
    plain = kernel == "plain"
    if dt == "f32" and not plain:
        pytest.skip("float32 runs on the plain kernel only")
    n_pages = 64
    c = build_cache_case(DT[dt], H, KV, hd, lens, page, rows_cap, n_pages, 50)
    scale = 1.0 / math.sqrt(hd * 0.9)
    q_ref, k_ref = c["q"].cpu().clone(), c["k"].cpu().clone()
    pools_ref = [torch.zeros(n_pages, KV, page, hd, dtype=DT[dt]) for _ in range(2)]
    ref_ops.rope_kv_write(q_ref, k_ref, c["v"].cpu(), H, KV, hd, c["inv_freq"], hd, c["row_seq"], c["row_pos"],
                          c["new_len"], c["table"], pools_ref[0], pools_ref[1], rows_cap)
    ref = ref_ops.attention_prefill(q_ref, k_ref, c["v"].cpu(), H, KV, hd, c["cu"], max(lens), scale, cap, window, torch.float32)
    # what earlier steps left: positions below `starts`, written as one step per sequence set
    pools = [torch.full((n_pages, KV, page, hd), 7.0, dtype=DT[dt], device=DEV) for _ in range(2)]
    first = torch.cat([torch.arange(int(c["cu"][i]), int(c["cu"][i]) + s) for i, s in enumerate(starts)]).long()
    if first.numel():
        ops.rope_kv_write(c["q"][first.to(DEV)].contiguous(), c["k"][first.to(DEV)].contiguous(), c["v"][first.to(DEV)].contiguous(),
                          H, KV, hd, c["inv_freq"].to(DEV), hd, c["row_seq"][first].to(DEV), c["row_pos"][first].to(DEV),
                          torch.tensor(starts, dtype=torch.int32, device=DEV), c["table"].to(DEV), pools[0], pools[1], rows_cap)
    # the step: positions starts[i] .. lens[i] - 1 of every sequence
    counts = [n - s for n, s in zip(lens, starts)]
    rows = torch.cat([torch.arange(int(c["cu"][i]) + s, int(c["cu"][i + 1])) for i, s in enumerate(starts)]).long()
    q, k, v = (c[name][rows.to(DEV)].contiguous() for name in ("q", "k", "v"))
    cu = torch.tensor([0] + list(torch.tensor(counts).cumsum(0)), dtype=torch.int32, device=DEV)
    row_seq, row_pos, new_len, table = (c[name].to(DEV) for name in ("row_seq", "row_pos", "new_len", "table"))
    row_seq, row_pos = row_seq[rows.to(DEV)].contiguous(), row_pos[rows.to(DEV)].contiguous()
    ops.force_plain_attention = plain
    try:
        ops.rope_kv_write(q, k, v, H, KV, hd, c["inv_freq"].to(DEV), hd, row_seq, row_pos, new_len, table, pools[0], pools[1],
                          rows_cap, write=False)
        before = [p.clone() for p in pools]
        got = ops.attention_prefill(q, k, v, H, KV, hd, cu, max(counts), scale, cap, window, DT[dt],
                                    row_seq=row_seq, row_pos=row_pos, cached=(new_len, table, pools[0], pools[1], rows_cap),
                                    shape=0 if plain else kernel)
        assert all(torch.equal(a, b) for a, b in zip(before, pools))       # neither the rotation nor the attention cached anything
        ops.kv_write(k, v, KV, hd, row_seq, row_pos, new_len, table, pools[0], pools[1], rows_cap)
    finally:
        ops.force_plain_attention = False
    assert rel_l2(got, ref[rows]) < (3e-6 if dt == "f32" else 8e-3)
    worst = max(rel_l2(got[i], ref[rows][i]) for i in range(0, len(rows), max(1, len(rows) // 50)))
    assert worst < (1e-5 if dt == "f32" else 3e-2)
    # the cache afterwards: every row a whole-sequence step writes holds the same values
    written = (pools_ref[0] != 0).any(dim=-1)
    t = 3e-6 if dt == "f32" else 6e-3
    assert rel_l2(pools[0].cpu()[written], pools_ref[0][written]) < t
    assert torch.equal(pools[1].cpu()[written], pools_ref[1][written])
    assert bool((pools[0].cpu()[~written] == 7.0).all())


@pytest.mark.parametrize("plain", [True, False])
@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("H,KV,hd,lens,page,window,rows_cap,cap", ATTN_CASES)
def test_attention_decode(ops, plain, dt, H, KV, hd, lens, page, window, rows_cap, cap):
    if dt == "f32" and not plain:
        pytest.skip("float32 runs on the plain kernel only")
    n_pages = 24
    c = build_cache_case(DT[dt], H, KV, hd, lens, page, rows_cap, n_pages, 40)
    pools_ref = [torch.zeros(n_pages, KV, page, hd, dtype=DT[dt]) for _ in range(2)]
    # stale rows of an earlier occupant must not leak: fill the pools with large values first
    for p in pools_ref:
        p.fill_(7.0)
    ref_ops.rope_kv_write(c["q"].cpu().clone(), c["k"].cpu().clone(), c["v"].cpu(), H, KV, hd, None, 0, c["row_seq"],
                          c["row_pos"], c["new_len"], c["table"], pools_ref[0], pools_ref[1], rows_cap)
    qlast = torch.stack([c["q"].cpu()[int(c["cu"][i + 1]) - 1] for i in range(len(lens))]).contiguous()
    scale = 1.0 / math.sqrt(hd * 1.3)
    ref = ref_ops.attention_decode(qlast, H, KV, hd, c["new_len"], c["table"], pools_ref[0], pools_ref[1], rows_cap, scale,
                                   cap, window, torch.float32)
    ops.force_plain_attention = plain
    try:
        got = ops.attention_decode(qlast.to(DEV), H, KV, hd, c["new_len"].to(DEV), c["table"].to(DEV),
                                   pools_ref[0].to(DEV), pools_ref[1].to(DEV), rows_cap, scale, cap, window, DT[dt],
                                   max_keys=max(lens))
        if not plain:
            for splits in (1, 2, 5):
                again = ops.attention_decode(qlast.to(DEV), H, KV, hd, c["new_len"].to(DEV), c["table"].to(DEV),
                                             pools_ref[0].to(DEV), pools_ref[1].to(DEV), rows_cap, scale, cap, window,
                                             DT[dt], max_keys=max(lens), splits=splits)
                assert rel_l2(again, ref) < 8e-3, splits
    finally:
        ops.force_plain_attention = False
    assert rel_l2(got, ref) < (3e-6 if dt == "f32" else 8e-3)


@pytest.mark.parametrize("splits", [None, 1, 3])
@pytest.mark.parametrize("slices", [0, 1, 3])
@pytest.mark.parametrize("H,KV,hd,lens,page,window,rows_cap,cap", ATTN_CASES)
def test_attention_decode_step(ops, splits, slices, H, KV, hd, lens, page, window, rows_cap, cap):
    """Rotation, cache write and attention of a decode step in one launch, against the three reference parts.  The
    cache holds every earlier position; the step's projections come as bf16 rows (slices 0) or as float32 K slices."""
    from trapetum_amd.kernels.ops import SplitRows
    n_pages, n = 24, len(lens)
    c = build_cache_case(torch.bfloat16, H, KV, hd, lens, page, rows_cap, n_pages, 70)
    rot = hd if hd != 80 else 48                            # one case with a rotation over part of the head
    inv_freq = c["inv_freq"][:rot // 2].contiguous()
    pools_ref = [torch.full((n_pages, KV, page, hd), 7.0, dtype=torch.bfloat16) for _ in range(2)]
    earlier = c["row_pos"] < (c["new_len"][c["row_seq"].long()] - 1)          # all rows but each sequence's last
    keep = earlier.nonzero().flatten()
    ref_ops.rope_kv_write(c["q"].cpu()[keep].clone(), c["k"].cpu()[keep].clone(), c["v"].cpu()[keep], H, KV, hd, inv_freq, rot,
                          c["row_seq"][keep], c["row_pos"][keep], c["new_len"] - 1, c["table"], pools_ref[0], pools_ref[1], rows_cap)
    pools = [p.to(DEV) for p in pools_ref]
    last = torch.tensor([int(c["cu"][i + 1]) - 1 for i in range(n)])
    qkv = torch.cat([c["q"].cpu()[last], c["k"].cpu()[last], c["v"].cpu()[last]], dim=1).float()
    if slices:
        parts = torch.randn(slices, *qkv.shape, generator=torch.Generator().manual_seed(71))
        parts[0] += qkv - parts.sum(0)
        given, summed = SplitRows(parts.contiguous().to(DEV)), parts[0].clone()
        for sl in range(1, slices):
            summed += parts[sl]
    else:
        given, summed = qkv.to(torch.bfloat16).to(DEV), qkv.to(torch.bfloat16).float()
    scale = 1.0 / math.sqrt(hd * 1.3)
    ref = ref_ops.attention_decode_step(summed, H, KV, hd, inv_freq, rot, c["new_len"], c["table"], pools_ref[0], pools_ref[1],
                                        rows_cap, scale, cap, window, torch.float32)
    if not ops.fuses_decode_step(torch.bfloat16, H, KV, hd, pools[0]):
        assert H // KV > 16
        pytest.skip("more than 16 query heads per kv head run on the separate kernels")
    got = ops.attention_decode_step(given, H, KV, hd, inv_freq.to(DEV), rot, c["new_len"].to(DEV), c["table"].to(DEV),
                                    pools[0], pools[1], rows_cap, scale, cap, window, torch.bfloat16, max_keys=max(lens),
                                    splits=splits)
    assert rel_l2(got, ref) < 8e-3
    assert rel_l2(pools[0], pools_ref[0]) < 6e-3 and rel_l2(pools[1], pools_ref[1]) < 6e-3
    assert torch.equal((pools[0].cpu() != 7.0).any(dim=-1), (pools_ref[0] != 7.0).any(dim=-1))      # no other row touched
    # queries only, on a cache that another run filled: the pools stay as they are
    before = [p.clone() for p in pools]
    got_q = ops.attention_decode_step(given.slices[..., :H * hd].contiguous() if slices else given[:, :H * hd].contiguous(),
                                      H, KV, hd, inv_freq.to(DEV), rot, c["new_len"].to(DEV), c["table"].to(DEV),
                                      pools[0], pools[1], rows_cap, scale, cap, window, torch.bfloat16, max_keys=max(lens),
                                      write_kv=False, splits=splits) if not slices else None
    if got_q is not None:
        assert rel_l2(got_q, ref) < 8e-3
        assert torch.equal(before[0], pools[0]) and torch.equal(before[1], pools[1])


def test_attention_far_key_stands_out(ops):
    """One key among hundreds carries the answer: its score is made to dominate, so a kernel that drops
    or misplaces it (a chunk boundary, a page boundary) returns another value row."""
    H, KV, hd, n, page = 4, 2, 64, 700, 64
    for target in (0, 63, 64, 333, 699):
        c = build_cache_case(torch.bfloat16, H, KV, hd, (n,), page, 0, 16, 50 + target)
        k = c["k"].cpu().float().reshape(n, KV, hd) * 0.05
        q = torch.zeros(1, H, hd)
        q[0, :, :] = k[target, :, :].repeat_interleave(H // KV, dim=0) * 4000.0
        pools = [torch.zeros(16, KV, page, hd, dtype=torch.bfloat16) for _ in range(2)]
        kb = k.reshape(n, KV * hd).to(torch.bfloat16)
        ref_ops.rope_kv_write(torch.zeros(n, H * hd, dtype=torch.bfloat16), kb, c["v"].cpu(), H, KV, hd, None, 0,
                              c["row_seq"], c["row_pos"], c["new_len"], c["table"], pools[0], pools[1], 0)
        qb = q.reshape(1, H * hd).to(torch.bfloat16)
        for plain in (True, False):
            ops.force_plain_attention = plain
            try:
                got = ops.attention_decode(qb.to(DEV), H, KV, hd, c["new_len"].to(DEV), c["table"].to(DEV),
                                           pools[0].to(DEV), pools[1].to(DEV), 0, 1.0, 0.0, 0, torch.bfloat16, max_keys=n,
                                           splits=None if plain else 1 + target % 7)
            finally:
                ops.force_plain_attention = False
            want = c["v"].cpu().float().reshape(n, KV, hd)[target].repeat_interleave(H // KV, dim=0).reshape(1, H * hd)
            assert rel_l2(got, want) < 2e-2, (target, plain)


@pytest.mark.parametrize("window,rows_cap,lens", [(4096, 4096, (5000, 4100, 4096, 9000)), (0, 0, (5000, 8191, 63, 64)),
                                                  (1000, 1024, (1000, 1001, 3333, 2048))])
def test_attention_decode_long_contexts(ops, window, rows_cap, lens):
    """Thousands of keys at the 2B head size: rings that have wrapped once and twice, a window shorter than its ring,
    lengths at and beside a page's end, pages scattered over the pool, and every way of cutting the keys into slices."""
    H, KV, hd, page, scale, cap = 8, 4, 256, 64, 1 / 16.0, 50.0
    g = torch.Generator().manual_seed(5)
    n = len(lens)
    per = [-(-(min(l, rows_cap) if rows_cap else l) // page) for l in lens]
    n_pages = sum(per) + 3
    kp, vp = (torch.zeros(n_pages, KV, page, hd, dtype=torch.bfloat16) for _ in range(2))
    free = torch.randperm(n_pages, generator=g).tolist()
    table = torch.full((n, max(per)), -1, dtype=torch.int32)
    q = (torch.randn(n, H, hd, generator=g) * 0.5).to(torch.bfloat16)
    ref = torch.zeros(n, H, hd)
    for i, l in enumerate(lens):
        table[i, :per[i]] = torch.tensor([free.pop() for _ in range(per[i])], dtype=torch.int32)
        k = (torch.randn(l, KV, hd, generator=g) * 0.5).to(torch.bfloat16)
        v = torch.randn(l, KV, hd, generator=g).to(torch.bfloat16)
        kept = torch.arange(max(0, l - rows_cap) if rows_cap else 0, l)            # what the ring still holds
        rows = kept % rows_cap if rows_cap else kept
        pages = table[i].long()[rows // page]
        kp[pages, :, rows % page] = k[kept]
        vp[pages, :, rows % page] = v[kept]
        lo = max(0, l - window) if window else 0
        scores = torch.einsum("tgd,gqd->gqt", k[lo:].float(), q[i].float().reshape(KV, H // KV, hd)) * scale
        weights = torch.softmax(cap * torch.tanh(scores / cap), dim=-1)
        ref[i] = torch.einsum("gqt,tgd->gqd", weights, v[lo:].float()).reshape(H, hd)
    for splits in (None, 1, 7, 33, 128):
        got = ops.attention_decode(q.reshape(n, H * hd).to(DEV), H, KV, hd, torch.tensor(lens, dtype=torch.int32, device=DEV),
                                   table.to(DEV), kp.to(DEV), vp.to(DEV), rows_cap, scale, cap, window, torch.bfloat16,
                                   max_keys=max(lens), splits=splits)
        assert rel_l2(got.reshape(n, H, hd), ref) < 8e-3, splits


def test_argmax_ties_and_nan(ops):
    z = torch.full((3, 7001), -1.0)
    z[0, 100] = z[0, 7000] = 5.0               # tie: the smaller index wins (runtime/src/bin/opt_check.rs:37-65)
    z[1, 7000] = 2.0
    z[2, 0] = float("nan")
    z[2, 5] = 0.5
    assert ops.argmax(z.to(DEV)).tolist() == [100, 7000, 5]
    big = randn(5, 256000, seed=60)
    assert ops.argmax(big).tolist() == big.cpu().argmax(dim=-1).tolist()


# ---- token choice ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("vocab,temperature,top_k,top_p", [(256, 0.7, 256, 0.95), (7001, 1.0, 40, 1.0), (7001, 0.3, 1000, 0.5),
                                                           (256000, 0.9, 256, 0.95), (513, 1.5, 1, 1.0), (513, 0.8, 600, 0.99), (513, 0.8, 0, 1.0),
                                                           (50001, 1.2, 0, 1.0)])
def test_sample_follows_the_plain_sampler(ops, vocab, temperature, top_k, top_p):
    """Sort by logit (ties: smaller id), keep top_k, softmax at the temperature, shortest prefix reaching top_p, walk
    with u (runtime/src/bin/serve.rs:41-72).  Ties and a dominant token are planted; where the uniform number falls
    within float32 rounding of a boundary of the walk either neighbour is right."""
    rows = 6
    z = randn(rows, vocab, seed=80, scale=3.0).cpu()
    z[1, 5] = z[1, 77] = z[1].max() + 1.0                    # a tie at the top
    z[2, vocab - 1] = z[2].max() + 30.0                      # one token takes all the mass
    u = torch.tensor([0.0, 0.5, 0.999, 0.25, 0.75, 0.9999], dtype=torch.float32)
    with pytest.raises(Exception, match="top_k"):            # the kernel sorts at most 1024 candidates and says so
        ops.sample(z.to(DEV), temperature, 2000, top_p, u.to(DEV))
    with pytest.raises(Exception, match="nucleus"):          # the whole vocabulary (top_k 0) goes without a nucleus
        ops.sample(z.to(DEV), temperature, 0, 0.9, u.to(DEV))
    got = ops.sample(z.to(DEV), temperature, top_k, top_p, u.to(DEV)).cpu().tolist()
    for b in range(rows):
        choices = set()
        for du in (-2e-6, 0.0, 2e-6):
            ub = min(max(float(u[b]) + du, 0.0), 0.9999999)
            choices.add(int(ref_ops.sample(z[b:b + 1], temperature, top_k, top_p, torch.tensor([ub]))[0]))
        assert got[b] in choices, (b, got[b], choices)
    assert got[2] == vocab - 1


def test_recent_push(ops):
    """A row's id goes to the place its cursor names, the cursor moves on and wraps at the ring's end."""
    ring = torch.full((3, 5), -1, dtype=torch.int32, device=DEV)
    cursor = torch.tensor([0, 4, 2], dtype=torch.int32, device=DEV)
    ops.recent_push(torch.tensor([7, 8, 9], dtype=torch.int32, device=DEV), ring, cursor)
    ops.recent_push(torch.tensor([1, 2, 3], dtype=torch.int32, device=DEV), ring, cursor)
    assert ring.cpu().tolist() == [[7, 1, -1, -1, -1], [2, -1, -1, -1, 8], [-1, -1, 9, 3, -1]]
    assert cursor.cpu().tolist() == [2, 1, 4]


@pytest.mark.parametrize("vocab,window", [(256, 8), (256000, 128)])
def test_repetition_penalty(ops, vocab, window):
    """Each distinct recent token once: z / penalty if z > 0 else z * penalty (runtime/src/bin/serve.rs:1330-1340)."""
    z = randn(3, vocab, seed=81, scale=2.0)
    recent = torch.full((3, window), -1, dtype=torch.int32)
    recent[0, :4] = torch.tensor([3, 3, 9, vocab - 1])       # a token twice in the window is penalised once
    recent[1, :] = torch.arange(window) * 2 % vocab
    ref = z.cpu().clone()
    ref_ops.apply_repetition_penalty(ref, recent, 1.3)
    ops.apply_repetition_penalty(z, recent.to(DEV), 1.3)
    assert torch.allclose(z.cpu(), ref, rtol=1e-6, atol=0)
    untouched = z.cpu().clone()
    ops.apply_repetition_penalty(z, recent.to(DEV), 1.0)     # 1.0 switches it off
    assert torch.equal(z.cpu(), untouched)
