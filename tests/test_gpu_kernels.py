"""Each HIP kernel alone against its plain torch reference (tests/torch_ops.py), at sizes other than the engine's
tiny configurations: widths and vocabularies that are no power of two, odd head counts and groups, page edges."""
import math
import random
from types import SimpleNamespace

import pytest
import torch

pytestmark = pytest.mark.gpu

from torch_ops import TorchOps

DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


@pytest.fixture(scope="module")
def ops_for():
    from tiny_inference_server_amd.ops.hip_ops import HipOps
    made = {}

    def get(dtype):
        if dtype not in made:
            made[dtype] = HipOps("cuda:0", dtype)
        return made[dtype]
    return get


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(shape, generator=g)).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,D", [(1, 8), (7, 1536), (33, 1000), (3, 5000), (70, 1536), (35, 4096), (33, 4104), (41, 64)])
def test_rmsnorm(ops_for, dtype, rows, D):
    ops, ref = ops_for(dtype), TorchOps(dtype=dtype)
    x = rnd((rows, D), dtype, 1, 3.0)
    x[0] = 0                                   # an all-zero row gives 0, not NaN: eps sits outside the root
    gain = 1 + 0.1 * rnd((D,), torch.float32, 2)
    got = ops.rmsnorm(x.cuda(), gain.cuda(), 2e-8).cpu()
    assert torch.isfinite(got).all() and (got[0] == 0).all()
    torch.testing.assert_close(got.float(), ref.rmsnorm(x, gain, 2e-8).float(), **tol(dtype))
    # strided input and output: the middle columns of a wider buffer
    wide = rnd((rows, 2 * D), dtype, 3).cuda()
    out = torch.zeros(rows, 2 * D, dtype=dtype, device="cuda")
    ops.rmsnorm(wide[:, D:], gain.cuda(), 1e-5, out=out[:, :D])
    torch.testing.assert_close(out[:, :D].cpu().float(), ref.rmsnorm(wide[:, D:].cpu(), gain, 1e-5).float(), **tol(dtype))
    assert (out[:, D:] == 0).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_fused_norm_and_row_moves(ops_for, dtype):
    ops, ref = ops_for(dtype), TorchOps(dtype=dtype)
    V, D, n = 777, 200, 19
    table = rnd((V, D), dtype, 4)
    toks = torch.tensor([random.Random(5).randrange(V) for _ in range(n)], dtype=torch.int32)
    gain = 1 + 0.1 * rnd((D,), torch.float32, 6)
    assert torch.equal(ops.embedding(table.cuda(), toks.cuda()).cpu(), table[toks.long()])
    out = torch.zeros(n, 2 * D, dtype=dtype, device="cuda")
    ops.embedding_rmsnorm(table.cuda(), toks.cuda(), gain.cuda(), 1e-6, out=out[:, D:])
    torch.testing.assert_close(out[:, D:].cpu().float(), ref.embedding_rmsnorm(table, toks, gain, 1e-6).float(), **tol(dtype))
    # gather from rows or from state, then keep rows in state
    src, state = rnd((n, D), dtype, 7), rnd((6, D), dtype, 8)
    index = torch.tensor([3, -1, 0, -6, 18, 18, -2], dtype=torch.int32)
    got = ops.gather_rows(src.cuda(), state.cuda(), index.cuda()).cpu()
    assert torch.equal(got, ref.gather_rows(src, state, index))
    st_gpu = state.cuda()
    ops.copy_rows(src.cuda(), torch.tensor([4, 9], dtype=torch.int32).cuda(), st_gpu,
                  torch.tensor([5, 0], dtype=torch.int32).cuda())
    want = state.clone(); want[5] = src[4]; want[0] = src[9]
    assert torch.equal(st_gpu.cpu(), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,F", [(1, 176), (9, 4096), (5, 1001)])
def test_swiglu(ops_for, dtype, rows, F):
    ops, ref = ops_for(dtype), TorchOps(dtype=dtype)
    gu = rnd((rows, 2 * F), dtype, 9, 2.0)
    gu[:, 6] = 0                               # a zero gate (unit 3) gives a zero output whatever its up value is
    got = ops.swiglu(gu.cuda()).cpu()
    assert (got[:, 3] == 0).all()
    torch.testing.assert_close(got.float(), ref.swiglu(gu).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (5, 1000, 96), (70, 130, 257), (64, 2304, 1536), (3, 515, 512)])
def test_linear(ops_for, dtype, M, N, K):
    ops = ops_for(dtype)
    x, w, res = rnd((M, K), dtype, 10), rnd((N, K), dtype, 11, K ** -0.5), rnd((M, N), dtype, 12)
    want = x.double() @ w.double().t()
    t = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(ops.linear(x.cuda(), w.cuda()).cpu().double(), want, **t)
    torch.testing.assert_close(ops.linear(x.cuda(), w.cuda(), residual=res.cuda()).cpu().double(), want + res.double(), **t)
    lg = ops.linear(x.cuda(), w.cuda(), out_dtype=torch.float32)
    assert lg.dtype == torch.float32
    torch.testing.assert_close(lg.cpu().double(), want, **t)


def test_linear_32bit_is_true_32bit(ops_for):
    """Products of numbers that need 24 bits: a reduced-precision matrix mode (tf32-like, bf16 x3) would lose them."""
    ops = ops_for(torch.float32)
    K = 512
    x = (1 + torch.arange(K, dtype=torch.float64) * 2.0 ** -20).float().view(1, K)
    w = (1 - torch.arange(K, dtype=torch.float64) * 2.0 ** -21).float().view(1, K)
    want = (x.double() * w.double()).sum().item()
    got = ops.linear(x.cuda(), w.cuda()).item()
    assert abs(got - want) / want < 3e-7


def make_paged(kv_lens, n_kv, hd, page_size, dtype, seed, shuffle=True):
    """Keys and values of several requests scattered over shuffled pages (reference test_gqa_paged.py:15-28)."""
    n_pages = sum(-(-L // page_size) for L in kv_lens) + 3
    ids = list(range(n_pages))
    if shuffle:
        random.Random(seed).shuffle(ids)
    # unused slots hold NaN: a kernel that lets a masked slot into its arithmetic, even weighted by zero, shows it
    plane = torch.full((n_pages, 2, n_kv, page_size, hd), float("nan"), dtype=dtype)
    tables, ks, vs = [], [], []
    width = max(-(-L // page_size) for L in kv_lens)
    for i, L in enumerate(kv_lens):
        k, v = rnd((L, n_kv, hd), dtype, seed + 10 * i), rnd((L, n_kv, hd), dtype, seed + 10 * i + 1)
        pages = [ids.pop() for _ in range(-(-L // page_size))]
        for j in range(L):
            plane[pages[j // page_size], 0, :, j % page_size] = k[j]
            plane[pages[j // page_size], 1].view(n_kv, hd, page_size)[:, :, j % page_size] = v[j]     # values lie transposed
        tables.append(pages + [0] * (width - len(pages)))
        ks.append(k); vs.append(v)
    return plane, torch.tensor(tables, dtype=torch.int32), ks, vs


def dense_reference(q, k, v, group, pos, window=0):
    """One row: query heads [NH, hd] against keys [0, pos] by library attention on repeated kv heads
    (the reference's own oracle: test_gqa_paged.py:39-44)."""
    lo = max(0, pos - window + 1) if window else 0
    kq = k[lo:pos + 1].double().repeat_interleave(group, dim=1).transpose(0, 1)     # [NH, keys, hd]
    vq = v[lo:pos + 1].double().repeat_interleave(group, dim=1).transpose(0, 1)
    return torch.nn.functional.scaled_dot_product_attention(q.double()[:, None, :], kq, vq)[:, 0, :]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,page_size,kv_lens", [
    (8, 2, 64, 16, [37, 512, 2000]),           # the reference's case: test_gqa_paged.py:11-17
    (3, 1, 32, 8, [1, 9, 24, 40]),
    (6, 3, 48, 16, [16, 17, 300]),
    (12, 3, 128, 16, [4096, 130]),
    # lengths that differ a hundredfold in one step: every request gets splits by its own length
    (12, 3, 128, 16, [1, 5000, 17, 900, 33, 4096, 64, 2, 8100, 640, 31, 32, 2500, 7, 129, 1300]),
    (16, 4, 128, 16, [40 + 127 * i for i in range(64)]),
    (32, 8, 128, 16, [40 + 127 * i for i in range(64)]),      # too many key/value heads for a planned list: same splits for all
    (5, 5, 8, 4, [3, 1100]),
    (4, 1, 256, 32, [65]),
])
def test_paged_attention_single_rows(ops_for, dtype, n_heads, n_kv, hd, page_size, kv_lens):
    """Decode-like rows: the last position of several requests with scattered pages."""
    from tiny_inference_server_amd.ops import hip_ops
    ops = ops_for(dtype)
    group = n_heads // n_kv
    plane, tables, ks, vs = make_paged(kv_lens, n_kv, hd, page_size, dtype, seed=20)
    B = len(kv_lens)
    # which of these cases take the list planned request by request (bfloat16 only) is part of what is tested
    planned = hip_ops.uneven_lengths([(i, L - 1, 1) for i, L in enumerate(kv_lens)]) and hip_ops.planned_list_pays(B, n_kv)
    assert planned == (B >= 16 and n_kv < 8)
    q = rnd((B, n_heads * hd), dtype, 21)
    batch = SimpleNamespace(positions=torch.tensor([L - 1 for L in kv_lens], dtype=torch.int32).cuda(),
                            row_seq=torch.arange(B, dtype=torch.int32).cuda(),
                            block_tables={"g": tables.cuda()}, max_kv_len=max(kv_lens), extras={},
                            n_rows=B, max_seq_rows=1, seq_rows=[(i, kv_lens[i] - 1, 1) for i in range(B)])
    got = ops.paged_attention(q.cuda(), plane.cuda(), batch, "g", n_heads, n_kv, hd).cpu()
    t = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    for i, L in enumerate(kv_lens):
        want = dense_reference(q[i].view(n_heads, hd), ks[i], vs[i], group, L - 1)
        torch.testing.assert_close(got[i].view(n_heads, hd).double(), want, **t)
    if group > 1 and n_kv > 1:
        # negative control (reference test_gqa_paged.py:50-53): the wrong head mapping must not match
        bad = dense_reference(q[0].view(n_heads, hd), ks[0].flip(1), vs[0].flip(1), group, kv_lens[0] - 1)
        assert not torch.allclose(got[0].view(n_heads, hd).double(), bad, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("window", [1000, 500])
def test_single_rows_of_uneven_lengths_behind_a_window(ops_for, window):
    """Decoded tokens of requests that differ widely in length, in a layer that sees a window ending inside a page:
    the splits are planned from what each row sees (the window's keys), not from its request's length."""
    from tiny_inference_server_amd.ops import hip_ops
    ops = ops_for(torch.bfloat16)
    n_heads, n_kv, hd, page_size = 12, 3, 128, 16
    kv_lens = [1, 5000, 17, 900, 33, 4096, 64, 2, 8100, 640, 31, 32, 2500, 7, 129, 1300, 151, 999]
    seq_rows = [(i, L - 1, 1) for i, L in enumerate(kv_lens)]
    assert hip_ops.uneven_lengths(seq_rows, window) and hip_ops.planned_list_pays(len(kv_lens), n_kv)
    entries, _ = hip_ops.decode_items(seq_rows, n_heads, n_kv, hd, window=window)
    live = entries[entries[:, 0] >= 0]
    for i, L in enumerate(kv_lens):          # no row gets more splits than its window has steps of 32 keys
        steps = (L + 31 - (max(0, L - window) & ~31)) // 32
        assert 1 <= (live[live[:, 0] == i][:, 1] >> 16).max() <= steps
    plane, tables, ks, vs = make_paged(kv_lens, n_kv, hd, page_size, torch.bfloat16, seed=27)
    B = len(kv_lens)
    q = rnd((B, n_heads * hd), torch.bfloat16, 28)
    batch = SimpleNamespace(positions=torch.tensor([L - 1 for L in kv_lens], dtype=torch.int32).cuda(),
                            row_seq=torch.arange(B, dtype=torch.int32).cuda(),
                            block_tables={"g": tables.cuda()}, max_kv_len=max(kv_lens), extras={},
                            n_rows=B, max_seq_rows=1, seq_rows=seq_rows)
    got = ops.paged_attention(q.cuda(), plane.cuda(), batch, "g", n_heads, n_kv, hd, window=window).cpu()
    for i, L in enumerate(kv_lens):
        want = dense_reference(q[i].view(n_heads, hd), ks[i], vs[i], n_heads // n_kv, L - 1, window)
        torch.testing.assert_close(got[i].view(n_heads, hd).double(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("n_heads,n_kv,hd,window,tile_splits", [(12, 3, 128, 0, False), (12, 3, 128, 0, True), (8, 2, 64, 700, False)])
def test_decoded_rows_of_uneven_lengths_beside_a_portions_tiles(ops_for, monkeypatch, n_heads, n_kv, hd, window, tile_splits):
    """A step as serving brings them: a prompt's portion, which goes to tiles, in the middle of decoded tokens of
    requests that differ widely in length, whose key splits are then planned row by row although the step is not one
    of single rows alone. The planned entries name the rows' lines of the block table, which are no longer 0, 1, ...;
    partial results of both kernels share the workspace and the merge."""
    from tiny_inference_server_amd.ops import hip_ops
    monkeypatch.setattr(hip_ops, "_ATTN_PLANNED_BESIDE_FROM", 0.0)    # (whether or not the estimate says it pays here)
    if tile_splits:
        monkeypatch.setattr(hip_ops, "_tiles_cut_pays", lambda *a: True)
    ops = ops_for(torch.bfloat16)
    page_size = 16
    lens = [1, 5000, 17, 900, 33, 4096, 64, 2, 640]
    lens_after = [31, 32, 2500, 7, 129, 1300, 151, 999, 3000, 45]
    p0, n = 1000, 600                                            # the portion: request 9 of 19
    kv_lens = lens + [p0 + n] + lens_after
    seq_rows, first = [], 0
    for i, L in enumerate(kv_lens):
        rows = n if i == len(lens) else 1
        seq_rows.append((first, L - rows, rows))
        first += rows
    R = first
    group, cols = n_heads // n_kv, hip_ops.tile_columns(hd)
    nb, items, tiles, steps = hip_ops.attention_items(seq_rows, group, cols, n_kv)
    beside = hip_ops.planned_beside_tiles(seq_rows, items, tiles, steps, n_heads, n_kv, hd, window)
    assert beside is not None and len(tiles) == -(-n // (4 * (cols // group)))
    live = beside[0][beside[0][:, 0] >= 0]
    assert sorted(set(live[:, 3].tolist())) == [i for i in range(len(kv_lens)) if i != len(lens)]
    assert (live[:, 1] >> 16).max() > 1                           # some row is cut, so partial results are merged
    plane, tables, ks, vs = make_paged(kv_lens, n_kv, hd, page_size, torch.bfloat16, seed=29)
    positions, row_seq = [], []
    for i, (f, q0, rows) in enumerate(seq_rows):
        positions += list(range(q0, q0 + rows)); row_seq += [i] * rows
    q = rnd((R, n_heads * hd), torch.bfloat16, 30)
    batch = SimpleNamespace(positions=torch.tensor(positions, dtype=torch.int32).cuda(),
                            row_seq=torch.tensor(row_seq, dtype=torch.int32).cuda(),
                            block_tables={"g": tables.cuda()}, max_kv_len=max(kv_lens), extras={},
                            n_rows=R, max_seq_rows=n, seq_rows=seq_rows)
    got = ops.paged_attention(q.cuda(), plane.cuda(), batch, "g", n_heads, n_kv, hd, window=window).cpu()
    assert torch.isfinite(got.float()).all()
    for r in list(range(len(lens))) + list(range(len(lens), len(lens) + n, 7)) + list(range(len(lens) + n - 2, R)):
        want = dense_reference(q[r].view(n_heads, hd), ks[row_seq[r]], vs[row_seq[r]], group, positions[r], window)
        torch.testing.assert_close(got[r].view(n_heads, hd).double(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("page_size", [16, 32])
def test_single_rows_walking_a_long_context_without_splits(ops_for, monkeypatch, page_size):
    """With no key splits one wave walks a request's whole context alone: thousands of keys, hundreds of steps,
    ending mid-page."""
    from tiny_inference_server_amd.ops import hip_ops
    monkeypatch.setattr(hip_ops, "_ATTN_TARGET_WAVES", 1)
    ops = ops_for(torch.bfloat16)
    n_heads, n_kv, hd = 4, 2, 64
    kv_lens = [4097, 9000, 33]
    plane, tables, ks, vs = make_paged(kv_lens, n_kv, hd, page_size, torch.bfloat16, seed=25)
    B = len(kv_lens)
    q = rnd((B, n_heads * hd), torch.bfloat16, 26)
    batch = SimpleNamespace(positions=torch.tensor([L - 1 for L in kv_lens], dtype=torch.int32).cuda(),
                            row_seq=torch.arange(B, dtype=torch.int32).cuda(),
                            block_tables={"g": tables.cuda()}, max_kv_len=max(kv_lens), extras={},
                            n_rows=B, max_seq_rows=1, seq_rows=[(i, kv_lens[i] - 1, 1) for i in range(B)])
    got = ops.paged_attention(q.cuda(), plane.cuda(), batch, "g", n_heads, n_kv, hd).cpu()
    for i, L in enumerate(kv_lens):
        want = dense_reference(q[i].view(n_heads, hd), ks[i], vs[i], n_heads // n_kv, L - 1)
        torch.testing.assert_close(got[i].view(n_heads, hd).double(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,page_size", [(4, 2, 64, 16), (3, 1, 32, 8), (12, 3, 128, 16), (2, 2, 48, 16)])
def test_paged_attention_portions_and_window(ops_for, dtype, n_heads, n_kv, hd, page_size):
    """Rows of prompt portions that start anywhere, beside single rows; and a window that ends mid-page."""
    ops = ops_for(dtype)
    group = n_heads // n_kv
    kv_lens = [150, 77, 200, 5]
    plane, tables, ks, vs = make_paged(kv_lens, n_kv, hd, page_size, dtype, seed=30)
    # request 0: rows at positions 100..149; request 1: its last row; request 2: positions 0..199; request 3: 3..4
    segs = [(0, 100, 50), (1, 76, 1), (2, 0, 200), (3, 3, 2)]
    positions, row_seq, seq_rows = [], [], []
    for s, p0, n in segs:
        seq_rows.append((len(positions), p0, n))
        positions += list(range(p0, p0 + n)); row_seq += [s] * n
    R = len(positions)
    q = rnd((R, n_heads * hd), dtype, 31)
    batch = SimpleNamespace(positions=torch.tensor(positions, dtype=torch.int32).cuda(),
                            row_seq=torch.tensor(row_seq, dtype=torch.int32).cuda(),
                            block_tables={"g": tables.cuda()}, max_kv_len=max(kv_lens), extras={},
                            n_rows=R, max_seq_rows=200, seq_rows=seq_rows)
    t = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    for window in (0, 37):
        got = ops.paged_attention(q.cuda(), plane.cuda(), batch, "g", n_heads, n_kv, hd, window=window).cpu()
        for r in range(0, R, 7):
            want = dense_reference(q[r].view(n_heads, hd), ks[row_seq[r]], vs[row_seq[r]], group, positions[r], window)
            torch.testing.assert_close(got[r].view(n_heads, hd).double(), want, **t)


@pytest.mark.parametrize("n_heads,n_kv,hd,page_size", [(12, 3, 128, 16), (32, 8, 32, 16), (4, 2, 64, 32)])
def test_mixed_rows_with_key_splits_chosen_item_by_item(ops_for, n_heads, n_kv, hd, page_size):
    """A small batch of prompt rows and single rows far into long requests: the keys are cut into splits, every item
    takes as many as its own length deserves (some one, some many), and the merge reads each row's count. With 32
    heads the rows times heads pass the size at which the merge goes row by row."""
    ops = ops_for(torch.bfloat16)
    group = n_heads // n_kv
    kv_lens = [1500, 1340, 40, 9, 700]
    plane, tables, ks, vs = make_paged(kv_lens, n_kv, hd, page_size, torch.bfloat16, seed=33)
    # request 0: its last row; request 1: rows 1040..1339 (a portion deep into a prompt); request 2: a whole short
    # prompt; request 3: its last row, nine keys in all; request 4: its last row
    segs = [(0, 1499, 1), (1, 1040, 300), (2, 0, 40), (3, 8, 1), (4, 699, 1)]
    positions, row_seq, seq_rows = [], [], []
    for s_, p0, n in segs:
        seq_rows.append((len(positions), p0, n))
        positions += list(range(p0, p0 + n)); row_seq += [s_] * n
    R = len(positions)
    q = rnd((R, n_heads * hd), torch.bfloat16, 34)
    batch = SimpleNamespace(positions=torch.tensor(positions, dtype=torch.int32).cuda(),
                            row_seq=torch.tensor(row_seq, dtype=torch.int32).cuda(),
                            block_tables={"g": tables.cuda()}, max_kv_len=max(kv_lens), extras={},
                            n_rows=R, max_seq_rows=300, seq_rows=seq_rows)
    got = ops.paged_attention(q.cuda(), plane.cuda(), batch, "g", n_heads, n_kv, hd).cpu()
    for r in list(range(0, R, 11)) + [0, 1, 300, 301, 340, 341, R - 1]:
        want = dense_reference(q[r].view(n_heads, hd), ks[row_seq[r]], vs[row_seq[r]], group, positions[r])
        torch.testing.assert_close(got[r].view(n_heads, hd).double(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("n_heads,n_kv,hd,page_size,window", [
    (12, 3, 128, 16, 0), (12, 3, 128, 16, 100), (4, 4, 64, 16, 0), (6, 2, 48, 32, 0), (16, 2, 32, 48, 45),
    (2, 1, 256, 16, 0), (5, 1, 16, 16, 33), (20, 1, 32, 16, 0)])
@pytest.mark.parametrize("splits", [False, True])
def test_long_portions_by_tiles(ops_for, monkeypatch, n_heads, n_kv, hd, page_size, window, splits):
    """Portions long enough for the workgroup kernel (tiles of rows whose four waves share each step's keys through
    LDS), beside rows that stay with the one-wave kernel: a whole prompt that ends mid-tile and mid-page, a portion
    deep into a long request, a decoded token and a three-row portion. Once as planned (chains this short are not
    cut), once with the tiles cut into key splits and merged, as those of long prompts are. Group sizes that divide a
    wave's 32 columns and ones that do not, head sizes in steps of 16 and of 32."""
    from tiny_inference_server_amd.ops import hip_ops
    from tiny_inference_server_amd.ops.hip_ops import attention_items, tile_columns
    if splits:
        monkeypatch.setattr(hip_ops, "_tiles_cut_pays", lambda *a: True)
    ops = ops_for(torch.bfloat16)
    group = n_heads // n_kv
    tile_rows = 4 * (tile_columns(hd) // group)
    n0, n1 = 2 * tile_rows + tile_rows // 2 + 5, tile_rows + 3
    kv_lens = [n0, 1000 + n1, 700, 12]
    segs = [(0, 0, n0), (1, 1000, n1), (2, 699, 1), (3, 9, 3)]
    plane, tables, ks, vs = make_paged(kv_lens, n_kv, hd, page_size, torch.bfloat16, seed=36)
    positions, row_seq, seq_rows = [], [], []
    for s_, p0, n in segs:
        seq_rows.append((len(positions), p0, n))
        positions += list(range(p0, p0 + n)); row_seq += [s_] * n
    R = len(positions)
    _, items, tiles, _ = attention_items(seq_rows, group, tile_columns(hd))
    short_too = 3 >= max(2, tile_rows // 2)
    assert len(tiles) == -(-n0 // tile_rows) + -(-n1 // tile_rows) + short_too and len(items) >= 1   # both kernels run
    q = rnd((R, n_heads * hd), torch.bfloat16, 37)
    batch = SimpleNamespace(positions=torch.tensor(positions, dtype=torch.int32).cuda(),
                            row_seq=torch.tensor(row_seq, dtype=torch.int32).cuda(),
                            block_tables={"g": tables.cuda()}, max_kv_len=max(kv_lens), extras={},
                            n_rows=R, max_seq_rows=n0, seq_rows=seq_rows)
    got = ops.paged_attention(q.cuda(), plane.cuda(), batch, "g", n_heads, n_kv, hd, window=window).cpu()
    assert torch.isfinite(got.float()).all()
    step = max(1, R // 60)
    for r in sorted(set(list(range(0, R, step)) + [0, 1, 15, 16, tile_rows - 1, tile_rows, n0 - 1, n0, n0 + 1, R - 5, R - 4, R - 1])):
        want = dense_reference(q[r].view(n_heads, hd), ks[row_seq[r]], vs[row_seq[r]], group, positions[r], window)
        torch.testing.assert_close(got[r].view(n_heads, hd).double(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("first", [0, 30, 60, 90])
def test_paged_attention_of_drawn_batches(ops_for, monkeypatch, first):
    """Thirty batches a case with everything drawn at random: heads and groups, head sizes in steps of 16 up to 256,
    the page, a window or none, and one to four requests (decoded tokens, short and long portions, from an empty
    cache or deep in a request) or ten to twenty-four decoded tokens of uneven lengths; and, drawn too, whether
    tiles' key ranges are cut however short, whether decoded rows beside tiles get planned splits, and whether short
    portions beside deep rows still go to tiles. Rows at the starts, middles and ends of portions, at tile and page
    edges and thirty drawn ones are compared with library attention over each row's own keys."""
    from tiny_inference_server_amd.ops import hip_ops
    ops = ops_for(torch.bfloat16)
    for case in range(first, first + 30):
        rng = random.Random(case)
        n_kv, group = rng.choice([1, 1, 2, 3, 4]), rng.choice([1, 2, 3, 4, 4, 5, 8])
        hd = rng.choice([16, 32, 48, 64, 80, 96, 128, 128, 160, 256])
        page = rng.choice([16, 16, 32, 48, 64])
        window = rng.choice([0, 0, 0, rng.randint(5, 900)])
        n_heads = n_kv * group
        n_req = rng.randint(1, 4) if rng.random() < 0.8 else rng.randint(10, 24)
        segs = []
        for i in range(n_req):
            kind = rng.random()
            if n_req > 4:
                n, p0 = 1, (rng.randint(0, 1500) if rng.random() < 0.7 else rng.randint(0, 40))
            elif kind < 0.3:
                n, p0 = 1, rng.randint(0, 2500)
            elif kind < 0.5:
                n, p0 = rng.randint(2, 40), rng.randint(0, 1500)
            elif kind < 0.8:
                n, p0 = rng.randint(41, 700), rng.choice([0, 0, rng.randint(1, 1500)])
            else:
                n, p0 = rng.randint(700, 1500), rng.choice([0, rng.randint(1, 800)])
            segs.append((i, p0, n))
        with monkeypatch.context() as m:
            if rng.random() < 0.4:
                m.setattr(hip_ops, "_tiles_cut_pays", lambda *a: True)
            if rng.random() < 0.5:
                m.setattr(hip_ops, "_ATTN_PLANNED_BESIDE_FROM", 0.0)
            if rng.random() < 0.5:
                m.setattr(hip_ops, "_ATTN_TILE_MIN_WORK_MIXED", 0)
            kv_lens = [p0 + n for _, p0, n in segs]
            plane, tables, ks, vs = make_paged(kv_lens, n_kv, hd, page, torch.bfloat16, seed=case * 7 + 1)
            positions, row_seq, seq_rows = [], [], []
            for s_, p0, n in segs:
                seq_rows.append((len(positions), p0, n))
                positions += list(range(p0, p0 + n)); row_seq += [s_] * n
            R = len(positions)
            q = rnd((R, n_heads * hd), torch.bfloat16, case * 7 + 2)
            batch = SimpleNamespace(positions=torch.tensor(positions, dtype=torch.int32).cuda(),
                                    row_seq=torch.tensor(row_seq, dtype=torch.int32).cuda(),
                                    block_tables={"g": tables.cuda()}, max_kv_len=max(kv_lens), extras={},
                                    n_rows=R, max_seq_rows=max(n for _, _, n in segs), seq_rows=seq_rows)
            got = ops.paged_attention(q.cuda(), plane.cuda(), batch, "g", n_heads, n_kv, hd, window=window).cpu()
        what = f"case {case}: heads {n_heads}/{n_kv} of {hd}, page {page}, window {window}, (first, rows) {[s[1:] for s in segs]}"
        assert torch.isfinite(got.float()).all(), what
        rows = set(rng.sample(range(R), min(R, 30)))
        for start, p0, n in seq_rows:
            rows |= {start, start + n - 1, start + n // 2} | {start + e for e in (15, 16, 31, 32, 63, 64, 127, 128) if e < n}
        for r in sorted(rows):
            want = dense_reference(q[r].view(n_heads, hd), ks[row_seq[r]], vs[row_seq[r]], group, positions[r], window)
            torch.testing.assert_close(got[r].view(n_heads, hd).double(), want, rtol=2e-2, atol=2e-2,
                                       msg=lambda m_: f"{what}, row {r} at position {positions[r]}: {m_}")


@pytest.mark.parametrize("splits", [False, True])
def test_a_tile_sees_a_far_key_and_a_rows_own_key(ops_for, monkeypatch, splits):
    """Two scores are made to stand out in a long portion: a key far back (in an early split of the tile's keys, when
    they are cut) for one row, and for another row the key at its own position, the last one the causal mask lets
    through."""
    from tiny_inference_server_amd.ops import hip_ops
    if splits:
        monkeypatch.setattr(hip_ops, "_tiles_cut_pays", lambda *a: True)
    ops = ops_for(torch.bfloat16)
    n_heads, n_kv, hd, page_size, L = 4, 1, 64, 16, 1200
    plane, tables, ks, vs = make_paged([L], n_kv, hd, page_size, torch.bfloat16, seed=38)
    p0, n = 900, 300
    q = rnd((n, n_heads * hd), torch.bfloat16, 39)
    for row, key in ((250, 3), (250, 1150), (77, 977), (77, 978)):
        k = ks[0].clone()
        k[key, 0] = (q[row].view(n_heads, hd)[0] * 4).to(torch.bfloat16)
        pl = plane.clone()
        pl[tables[0, key // page_size].item(), 0, 0, key % page_size] = k[key, 0]
        batch = SimpleNamespace(positions=torch.arange(p0, p0 + n, dtype=torch.int32).cuda(),
                                row_seq=torch.zeros(n, dtype=torch.int32).cuda(), block_tables={"g": tables.cuda()},
                                max_kv_len=L, extras={}, n_rows=n, max_seq_rows=n, seq_rows=[(0, p0, n)])
        got = ops.paged_attention(q.cuda(), pl.cuda(), batch, "g", n_heads, n_kv, hd).cpu()
        want = dense_reference(q[row].view(n_heads, hd), k, vs[0], n_heads, p0 + row)
        torch.testing.assert_close(got[row].view(n_heads, hd).double(), want, rtol=2e-2, atol=2e-2)
        seen = key <= p0 + row
        assert ((got[row].view(n_heads, hd)[0].double() - vs[0][key, 0].double()).abs().max() < 0.05) == seen


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_one_far_key_among_hundreds(ops_for, dtype):
    """One key far back is made to dominate: a kernel that skips a page or a split would miss it."""
    ops = ops_for(dtype)
    n_heads, n_kv, hd, page_size, L = 4, 2, 64, 16, 900
    plane, tables, ks, vs = make_paged([L], n_kv, hd, page_size, dtype, seed=40)
    q = rnd((1, n_heads * hd), dtype, 41)
    for far in (0, 15, 16, 511, 512, 899):
        k, v = ks[0].clone(), vs[0].clone()
        k[far] = (q.view(n_heads, hd)[::2] * 4).to(dtype)            # aligned with the query of each kv head's first q head
        page = tables[0, far // page_size].item()
        pl = plane.clone()
        pl[page, 0, :, far % page_size] = k[far]
        batch = SimpleNamespace(positions=torch.tensor([L - 1], dtype=torch.int32).cuda(),
                                row_seq=torch.zeros(1, dtype=torch.int32).cuda(), block_tables={"g": tables.cuda()},
                                max_kv_len=L, extras={}, n_rows=1, max_seq_rows=1, seq_rows=[(0, L - 1, 1)])
        got = ops.paged_attention(q.cuda(), pl.cuda(), batch, "g", n_heads, n_kv, hd).cpu().view(n_heads, hd)
        want = dense_reference(q.view(n_heads, hd), k, v, 2, L - 1)
        t = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
        torch.testing.assert_close(got.double(), want, **t)
        # the dominated heads return (almost) the far value itself
        assert (got[0].double() - v[far, 0].double()).abs().max() < 0.05


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,page_size,interleaved", [(8, 2, 8, 16, False), (3, 1, 32, 8, False),
                                                                    (12, 3, 128, 16, False), (4, 2, 48, 4, True)])
def test_rope_and_cache_write(ops_for, dtype, n_heads, n_kv, hd, page_size, interleaved):
    ops, ref = ops_for(dtype), TorchOps(dtype=dtype)
    n, n_pages, max_ctx = 23, 9, 300
    j = torch.arange(hd // 2)
    theta = 1.0 / torch.pow(torch.tensor(500000.0), (2 * j.float()) / hd)
    ang = torch.outer(torch.arange(max_ctx).float(), theta)
    table = torch.stack((torch.cos(ang), torch.sin(ang)), -1).contiguous()
    qkv = rnd((n, (n_heads + 2 * n_kv) * hd), dtype, 50)
    positions = torch.tensor(random.Random(51).sample(range(max_ctx), n), dtype=torch.int32)
    slots = torch.tensor(random.Random(52).sample(range(n_pages * page_size), n), dtype=torch.int32)
    plane0 = rnd((n_pages, 2, n_kv, page_size, hd), dtype, 53)
    a, pa = qkv.clone().cuda(), plane0.clone().cuda()
    ops.rope_write_kv(a, positions.cuda(), slots.cuda(), table.cuda(), pa, n_heads, n_kv, hd, page_size, interleaved)
    b, pb = qkv.clone(), plane0.clone()
    ref.rope_write_kv(b, positions, slots, table, pb, n_heads, n_kv, hd, page_size, interleaved)
    t = tol(dtype)
    torch.testing.assert_close(a.cpu()[:, :n_heads * hd].float(), b[:, :n_heads * hd].float(), **t)
    torch.testing.assert_close(pa.cpu().float(), pb.float(), **t)
    # position 0 is the identity; a unit vector at position 1 lands on cos 1 and sin 1 of its pair
    one = torch.zeros(2, (n_heads + 2 * n_kv) * hd, dtype=dtype)
    one[:, 0] = 1
    g = one.clone().cuda()
    ops.rope_write_kv(g, torch.tensor([0, 1], dtype=torch.int32).cuda(), slots[:2].cuda(), table.cuda(), pa, n_heads,
                      n_kv, hd, page_size, interleaved)
    g = g.cpu().float()
    assert torch.equal(g[0], one[0].float())
    partner = 1 if interleaved else hd // 2
    assert abs(g[1, 0] - math.cos(1)) < 1e-2 and abs(g[1, partner] - math.sin(1)) < 1e-2
    # reading without writing leaves the cache alone
    before = pa.clone()
    ops.rope_write_kv(qkv.clone().cuda(), positions.cuda(), slots.cuda(), table.cuda(), pa, n_heads, n_kv, hd,
                      page_size, interleaved, write_cache=False)
    assert torch.equal(before, pa)


@pytest.mark.parametrize("n", [23, 64, 203])
@pytest.mark.parametrize("n_heads,n_kv,hd,page_size", [(12, 3, 128, 16), (3, 1, 64, 32), (5, 5, 48, 16), (2, 1, 256, 16)])
def test_rope_and_cache_write_of_pair_ordered_rows(ops_for, n_heads, n_kv, hd, page_size, n):
    """Rows as the fused q/k/v projection leaves them (the members of every rotary pair side by side): few rows, and
    enough for the kernel that takes sixteen rows a workgroup and turns the values through LDS. Slots are runs of
    consecutive positions that start mid-page, with one row out of line, as the rows of prompt portions are."""
    ops, ref = ops_for(torch.bfloat16), TorchOps(dtype=torch.bfloat16)
    dtype = torch.bfloat16
    n_pages, max_ctx = 40, 700
    j = torch.arange(hd // 2)
    theta = 1.0 / torch.pow(torch.tensor(10000.0), (2 * j.float()) / hd)
    ang = torch.outer(torch.arange(max_ctx).float(), theta)
    table = torch.stack((torch.cos(ang), torch.sin(ang)), -1).contiguous()
    qkv = rnd((n, (n_heads + 2 * n_kv) * hd), dtype, 54)
    first = 5
    positions = torch.arange(first, first + n, dtype=torch.int32)
    pages = random.Random(55).sample(range(n_pages), -(-(first + n) // page_size) + 1)
    slots = torch.tensor([pages[p // page_size] * page_size + p % page_size for p in positions.tolist()], dtype=torch.int32)
    slots[n // 2], positions[n // 2] = pages[-1] * page_size + 3, 650          # a row of another request in between
    plane0 = rnd((n_pages, 2, n_kv, page_size, hd), dtype, 56)
    for write_cache in (True, False):
        pa, pb = plane0.clone().cuda(), plane0.clone()
        qa = torch.zeros(n, n_heads * hd, dtype=dtype).cuda()
        qb = torch.zeros(n, n_heads * hd, dtype=dtype)
        ops.rope_write_kv(qkv.clone().cuda(), positions.cuda(), slots.cuda(), table.cuda(), pa, n_heads, n_kv, hd,
                          page_size, False, write_cache=write_cache, paired=True, q_out=qa)
        ref.rope_write_kv(qkv.clone(), positions, slots, table, pb, n_heads, n_kv, hd, page_size, False,
                          write_cache=write_cache, paired=True, q_out=qb)
        torch.testing.assert_close(qa.cpu().float(), qb.float(), **tol(dtype))
        torch.testing.assert_close(pa.cpu().float(), pb.float(), **tol(dtype))
        if not write_cache:
            assert torch.equal(pa.cpu(), plane0)


def assert_same_draws(ref, got, logits, temperature, top_k, top_p, pen, u, ctx_t, off, note=None):
    """The kernel's tokens against the plain sampler's. The draw inverts a cumulative sum in token order, which the
    kernel adds in 32-bit and the plain sampler in 64-bit: where the uniform number falls within 2e-6 of the whole
    mass from a token's edge, either neighbour is right, so a token must lie between the plain sampler's draws at
    u - 2e-6 and u + 2e-6 (the draw is monotone in u); everywhere else that is equality."""
    want = ref.sample(logits, temperature, top_k, top_p, pen, u, ctx_t, off).tolist()
    lo = ref.sample(logits, temperature, top_k, top_p, pen, (u - 2e-6).clamp(min=0.0), ctx_t, off).tolist()
    hi = ref.sample(logits, temperature, top_k, top_p, pen, (u + 2e-6).clamp(max=1.0), ctx_t, off).tolist()
    got = got.tolist()
    for r in range(len(got)):
        assert got[r] == want[r] or lo[r] <= got[r] <= hi[r], (note, r, got[r], want[r], lo[r], hi[r])
        if lo[r] == hi[r]:
            assert got[r] == want[r]


@pytest.fixture(params=[1, 0], ids=["registers", "general"])
def sampling_kernel(request, ops_for):
    """Both sampling kernels: the one that keeps a row in registers, and the general one alone."""
    ops = ops_for(torch.float32)
    ops.sampling.cdll.tis_sample_use_registers(request.param)
    yield ops
    ops.sampling.cdll.tis_sample_use_registers(1)


@pytest.mark.parametrize("V", [6, 100, 1000, 9001, 48000, 98304, 100003])
def test_sampling(sampling_kernel, V):
    ops, ref = sampling_kernel, TorchOps()
    n = 8
    logits = rnd((n, V), torch.float32, 60, 3.0)
    temperature = torch.tensor([0.0, 1.0, 0.8, 1.0, 0.9, 1.3, 1.0, 0.7])
    top_k = torch.tensor([0, 1, 0, 3, 50, 0, 0, 5], dtype=torch.int32)
    top_p = torch.tensor([0.0, 0.0, 0.0, 0.9, 0.95, 0.5, 0.0, 0.3])
    pen = torch.tensor([1.0, 1.0, 1.0, 1.0, 1.1, 1.0, 1.3, 2.0])
    ctx = [torch.tensor(random.Random(61 + i).choices(range(V), k=7), dtype=torch.int32) for i in range(n)]
    off = torch.tensor([0] + list(torch.tensor([len(c) for c in ctx]).cumsum(0)), dtype=torch.int32)
    ctx_t = torch.cat(ctx)
    for trial in range(6):
        u = torch.rand(n, generator=torch.Generator().manual_seed(70 + trial))
        got = ops.sample(logits.cuda(), temperature.cuda(), top_k.cuda(), top_p.cuda(), pen.cuda(), u.cuda(),
                         ctx_t.cuda(), off.cuda()).cpu()
        assert_same_draws(ref, got, logits, temperature, top_k, top_p, pen, u, ctx_t, off, trial)
    assert ops.argmax(logits.cuda()).cpu().tolist() == logits.argmax(-1).tolist()


@pytest.mark.parametrize("V", [1000, 48000])
def test_sampling_against_the_reference_rule(sampling_kernel, V):
    """The kernel's draws against the reference's rule itself, as the plain implementation states it from
    server.py:22-50 (sort, top-k cut, cumulative top-p cut that keeps the first token across p, softmax), and not
    against a restatement of the kernel's method: 16 rows of mixed temperature, top-k, top-p and repetition penalty,
    7 uniform numbers each. A draw within 2e-6 of a token's edge in the cumulative distribution may be either
    neighbour (the kernel sums in 32-bit)."""
    import plain_model as pm
    ops = sampling_kernel
    n = 16
    logits = rnd((n, V), torch.float32, 260, 3.0)
    rng = random.Random(261)
    temperature = [rng.choice((0.5, 0.8, 0.9, 1.0, 1.3)) for _ in range(n)]
    top_k = [rng.choice((0, 0, 2, 5, 50, 200)) for _ in range(n)]
    top_p = [rng.choice((0.0, 0.0, 0.3, 0.9, 0.95)) for _ in range(n)]
    pen = [rng.choice((1.0, 1.0, 1.1, 1.3, 2.0)) for _ in range(n)]
    top_k[0], top_p[0], pen[0] = 50, 0.95, 1.1                      # the reference's run defaults (server.py:515-516)
    temperature[0] = 0.9
    # contexts that hold the rows' likeliest tokens, so that the penalty moves the draw
    ctx = [sorted(set(torch.topk(logits[i], 6).indices.tolist() + rng.choices(range(V), k=9))) for i in range(n)]
    off = torch.tensor([0] + list(torch.tensor([len(c) for c in ctx]).cumsum(0)), dtype=torch.int32)
    ctx_t = torch.tensor([t for c in ctx for t in c], dtype=torch.int32)
    probs = [pm.sampling_probs(logits[i], temperature[i], top_k[i], top_p[i], pen[i], ctx[i]) for i in range(n)]
    as_t = lambda v, dt: torch.tensor(v, dtype=dt).cuda()
    strict = 0
    for trial in range(7):
        u = torch.rand(n, generator=torch.Generator().manual_seed(270 + trial))
        got = ops.sample(logits.cuda(), as_t(temperature, torch.float32), as_t(top_k, torch.int32), as_t(top_p, torch.float32),
                         as_t(pen, torch.float32), u.cuda(), ctx_t.cuda(), off.cuda()).cpu().tolist()
        for i in range(n):
            want = pm.pick_by_uniform(probs[i], float(u[i]))
            lo, hi = pm.pick_by_uniform(probs[i], max(0.0, float(u[i]) - 2e-6)), pm.pick_by_uniform(probs[i], min(1.0, float(u[i]) + 2e-6))
            assert got[i] == want or lo <= got[i] <= hi, (trial, i, got[i], want, temperature[i], top_k[i], top_p[i], pen[i])
            strict += lo == hi
            assert probs[i][got[i]] > 0
    assert strict >= 100


@pytest.mark.parametrize("V", [300, 48000])
def test_sampling_with_many_values_at_the_cut(sampling_kernel, V):
    """All logits equal: every value ties at any top-k cut, so all are kept and the draw is uniform over the
    vocabulary, token by token in order; a row with a few values above a plateau keeps those and the plateau."""
    ops, ref = sampling_kernel, TorchOps()
    n = 6
    logits = torch.zeros(n, V)
    logits[3:, :] = -1.0
    logits[3:, [7, V - 2, V // 2]] = torch.tensor([2.0, 1.0, 1.5])
    temperature = torch.tensor([1.0, 0.7, 1.0, 1.0, 0.9, 1.0])
    top_k = torch.tensor([50, 5, 2000 % V, 2, 50, 3], dtype=torch.int32)
    top_p = torch.zeros(n)           # (with ties a top-p cut is a matter of definition: the kernel keeps all of a tie)
    pen = torch.ones(n)
    for trial in range(4):
        u = torch.rand(n, generator=torch.Generator().manual_seed(170 + trial))
        got = ops.sample(logits.cuda(), temperature.cuda(), top_k.cuda(), top_p.cuda(), pen.cuda(), u.cuda()).cpu()
        assert_same_draws(ref, got, logits, temperature, top_k, top_p, pen, u, None, None, trial)


def test_sampling_reference_vectors(ops_for):
    """The reference's own vector (test_server.py:120-122): a repetition penalty pushes token 5 below token 7."""
    ops = ops_for(torch.float32)
    lg = torch.zeros(1, 100); lg[0, 5] = 5.0; lg[0, 7] = 4.9
    one = lambda v, dt=torch.float32: torch.tensor([v], dtype=dt).cuda()
    args = (one(1.0), one(1, torch.int32), one(0.0))
    assert ops.sample(lg.cuda(), *args, one(1.0), one(0.5)).item() == 5
    assert ops.sample(lg.cuda(), *args, one(2.0), one(0.5), one(5, torch.int32), torch.tensor([0, 1], dtype=torch.int32).cuda()).item() == 7


@pytest.mark.parametrize("M", [33, 64, 65, 200, 777])
@pytest.mark.parametrize("N,K", [(96, 64), (1000, 96), (2304, 1536)])
def test_product_with_norm_residual_and_gate_for_many_rows(ops_for, M, N, K):
    """More rows than a workgroup of the few-row kernel takes: panels of rows (any width), or, at a width from the
    library's list, separate kernels around the library's product. The results agree with the reference's order of
    operations (norm rounded to bfloat16, product, gating)."""
    ops, ref = ops_for(torch.bfloat16), TorchOps(dtype=torch.bfloat16)
    x, w, res = rnd((M, K), torch.bfloat16, 80, 2.0), rnd((N, K), torch.bfloat16, 81, K ** -0.5), rnd((M, N), torch.bfloat16, 82)
    gain = 1 + 0.1 * rnd((K,), torch.float32, 83)
    t = dict(rtol=2e-2, atol=2e-2)
    xn = ref.rmsnorm(x, gain, 1e-5).double()
    normed = ops.linear(x.cuda(), w.cuda(), rms=(gain.cuda(), 1e-5)).cpu()
    torch.testing.assert_close(normed.double(), xn @ w.double().t(), **t)
    torch.testing.assert_close(ops.linear(x.cuda(), w.cuda(), residual=res.cuda()).cpu().double(),
                               x.double() @ w.double().t() + res.double(), **t)
    lg = ops.linear(x.cuda(), w.cuda(), out_dtype=torch.float32)          # the output table's case: 32-bit sums kept
    assert lg.dtype == torch.float32
    torch.testing.assert_close(lg.cpu().double(), x.double() @ w.double().t(), rtol=1e-4, atol=1e-4)
    gu = (xn @ w.double().t()).to(torch.bfloat16).double()
    want = torch.nn.functional.silu(gu[:, 0::2]) * gu[:, 1::2]
    torch.testing.assert_close(ops.linear_swiglu(x.cuda(), w.cuda(), rms=(gain.cuda(), 1e-5)).cpu().double(), want,
                               rtol=3e-2, atol=3e-2)
    if (N, K) not in ops.library_widths or M <= ops.few_rows:
        # our own kernels: a row's result does not depend on its panel or on the other rows
        for r in (0, M // 2, M - 1):
            others = rnd((M, K), torch.bfloat16, 84, 3.0)
            shift = (M // 3) if r + M // 3 < M else 0             # the row moves to another panel where it can
            others[r + shift] = x[r]
            again = ops.linear(others.cuda(), w.cuda(), rms=(gain.cuda(), 1e-5)).cpu()
            assert torch.equal(again[r + shift], normed[r])


@pytest.mark.parametrize("M", [129, 200, 777, 2049])
@pytest.mark.parametrize("N,K", [(4, 16), (64, 8), (132, 72), (520, 1528), (1536, 640), (4096, 4096), (6148, 200), (8196, 264)])
def test_tiled_product_at_widths_the_library_is_not_used_at(ops_for, M, N, K):
    """Many rows at a width outside the library's list go to the tiled product of this repository: row and column
    counts that end inside a tile, a K that ends inside a step of 64 (down to a single piece of 8), tiles of 64, 128
    and (2,049 rows by 8,196 columns) 256 columns, with a residual that is the output itself or another tensor. Against exact sums of the same bfloat16
    operands; and a row's result does not depend on which tile or rows it shares."""
    from tiny_inference_server_amd.ops.hip_ops import product_route
    ops = ops_for(torch.bfloat16)
    assert product_route(M, N, K, True, False, ops.library_widths, ops.few_rows) == "tiles"
    x, w = rnd((M, K), torch.bfloat16, 60, 1.0), rnd((N, K), torch.bfloat16, 61, K ** -0.5)
    res = rnd((M, N), torch.bfloat16, 62)
    want = x.double() @ w.double().t()
    t = dict(rtol=8e-3, atol=4e-3)
    got = ops.linear(x.cuda(), w.cuda())
    torch.testing.assert_close(got.cpu().double(), want, **t)
    torch.testing.assert_close(ops.linear(x.cuda(), w.cuda(), residual=res.cuda()).cpu().double(), want + res.double(), **t)
    # the residual as the output's own memory
    out, xd, wd = res.clone().cuda(), x.cuda(), w.cuda()
    ops.gemm_tiles.tis_gemm_tiles(xd.data_ptr(), K, wd.data_ptr(), out.data_ptr(), N, out.data_ptr(), N, M, N, K, 0,
                                  ops._stream())
    torch.testing.assert_close(out.cpu().double(), want + res.double(), **t)
    # 32-bit results (the output table's logits for many rows): the sums as they are
    lg = ops.linear(xd, wd, out_dtype=torch.float32)
    assert lg.dtype == torch.float32
    torch.testing.assert_close(lg.cpu().double(), want, rtol=1e-4, atol=1e-4)
    # a row moved to another place among other rows gives the same bits
    others = rnd((M, K), torch.bfloat16, 63, 2.0)
    others[M - 1] = x[3]
    again = ops.linear(others.cuda(), w.cuda())
    assert torch.equal(again[M - 1].cpu(), got[3].cpu())


def test_library_product_at_listed_widths(ops_for):
    """Every width that may go to the library's product (ops/library_widths.json), at row counts as serving brings
    them: a few more than the few-row kernel takes, a portion beside decoded tokens, a prediction head's rows one
    short of a portion. Each runs at the rounded row count of library_rows; the rows asked for are compared with
    plain multiply-adds in 32-bit, and what lies behind the result's rows is the caller's and stays as it was."""
    from tiny_inference_server_amd.ops.hip_ops import library_rows, _ptr
    ops = ops_for(torch.bfloat16)
    for i, (N, K) in enumerate(sorted(ops.library_widths)):
        w = rnd((N, K), torch.bfloat16, 300 + i, K ** -0.5).cuda()
        for M in (129, 200, 1024, 2047, 2112) + ((4096,) if i % 4 == 0 else ()):
            x, res = rnd((M, K), torch.bfloat16, 400 + i).cuda(), rnd((M, N), torch.bfloat16, 500 + i).cuda()
            print(f"library product: rows {M} (asked {library_rows(M)}), out {N}, in {K}", flush=True)
            got = ops.linear(x, w, residual=res)
            want, res32 = torch.empty(M, N, dtype=torch.float32, device="cuda"), res.float()
            ops.gemm_plain.tis_gemm_plain(1, 0, _ptr(x), x.stride(0), _ptr(w), K, _ptr(res32), N, _ptr(want), N, M, N, K,
                                          ops._stream())
            torch.cuda.synchronize()
            torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2)
            assert got.shape == (M, N) and ops._holds_rows(got, library_rows(M))
    assert 0 < ops.gemm_library.cdll.tis_gemm_library_plans() <= 256


@pytest.mark.parametrize("M", [1, 4, 8, 9, 16, 17, 32, 33, 48, 64])
@pytest.mark.parametrize("N,K", [(96, 64), (1000, 96), (130, 264), (2304, 1536), (1536, 4096)])
def test_skinny_product_with_fused_norm_residual_and_gate(ops_for, M, N, K):
    """The few-row matrix-core product and what is fused around it, against the unfused plain computation."""
    ops, ref = ops_for(torch.bfloat16), TorchOps(dtype=torch.bfloat16)
    x, w, res = rnd((M, K), torch.bfloat16, 80, 2.0), rnd((N, K), torch.bfloat16, 81, K ** -0.5), rnd((M, N), torch.bfloat16, 82)
    gain = 1 + 0.1 * rnd((K,), torch.float32, 83)
    # the kernel's own rounding points, then exact arithmetic: the activations times the gain are rounded to
    # bfloat16, the row factor sqrt(K)/(||x||+eps) multiplies the 32-bit sums. Only the output's rounding is left,
    # so the comparison is tight (half a unit of bfloat16 is 0.4 % of a value).
    t = dict(rtol=8e-3, atol=2e-3)
    xb = (x.float() * gain).to(torch.bfloat16).double()
    mul = (K ** 0.5) / (x.double().norm(dim=-1, keepdim=True) + 1e-5)
    normed = (xb @ w.double().t()) * mul
    torch.testing.assert_close(ops.linear(x.cuda(), w.cuda(), rms=(gain.cuda(), 1e-5)).cpu().double(), normed, **t)
    # and that is the reference's norm followed by the product, up to bfloat16 rounding of the normed rows
    xn = ref.rmsnorm(x, gain, 1e-5).double()
    assert ((xn @ w.double().t()) - normed).abs().max() < 0.05
    torch.testing.assert_close(ops.linear(x.cuda(), w.cuda(), residual=res.cuda()).cpu().double(),
                               x.double() @ w.double().t() + res.double(), **t)
    lg = ops.linear(x.cuda(), w.cuda(), out_dtype=torch.float32)
    assert lg.dtype == torch.float32
    torch.testing.assert_close(lg.cpu().double(), x.double() @ w.double().t(), rtol=1e-4, atol=1e-4)   # 32-bit sums kept
    want = torch.nn.functional.silu(normed[:, 0::2]) * normed[:, 1::2]
    torch.testing.assert_close(ops.linear_swiglu(x.cuda(), w.cuda(), rms=(gain.cuda(), 1e-5)).cpu().double(), want, **t)
    # a row's result does not depend on the other rows of the batch, nor on which row of it it is
    both = ops.linear(x.cuda(), w.cuda(), rms=(gain.cuda(), 1e-5)).cpu()
    others = rnd((M, K), torch.bfloat16, 84, 3.0)
    others[M - 1] = x[0]
    assert torch.equal(ops.linear(others.cuda(), w.cuda(), rms=(gain.cuda(), 1e-5)).cpu()[M - 1], both[0])
    # and the two kernels (few rows of a narrow matrix; everything else) agree up to the order of their sums
    ops.gemm_skinny.cdll.tis_gemm_skinny_staged_always(1)
    try:
        staged = ops.linear(x.cuda(), w.cuda(), rms=(gain.cuda(), 1e-5)).cpu()
    finally:
        ops.gemm_skinny.cdll.tis_gemm_skinny_staged_always(0)
    torch.testing.assert_close(staged.double(), normed, **t)
    torch.testing.assert_close(staged.float(), both.float(), rtol=8e-3, atol=2e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M", [1, 5, 16, 27, 33, 64, 65, 200])
@pytest.mark.parametrize("n_heads,n_kv,hd,page_size,interleaved", [(8, 2, 8, 16, False), (3, 1, 32, 8, False),
                                                                    (12, 3, 128, 16, False), (4, 2, 48, 16, True)])
def test_projection_with_rotary_and_cache_write(ops_for, dtype, M, n_heads, n_kv, hd, page_size, interleaved):
    """q/k/v projection + rotary + cache write: one kernel for few bfloat16 rows, two otherwise; same results."""
    ops, ref = ops_for(dtype), TorchOps(dtype=dtype)
    # (the headline model's width for 33 and 64 rows of its geometry: four row blocks of the few-row kernel at a real size)
    K, n_pages, max_ctx = (1536 if hd == 128 and M in (33, 64) else 96), -(-M // page_size) + 3, 300
    N = (n_heads + 2 * n_kv) * hd
    j = torch.arange(hd // 2)
    ang = torch.outer(torch.arange(max_ctx).float(), 1.0 / torch.pow(torch.tensor(1e4), (2 * j.float()) / hd))
    table = torch.stack((torch.cos(ang), torch.sin(ang)), -1).contiguous()
    x, w = rnd((M, K), dtype, 84), rnd((N, K), dtype, 85, K ** -0.5)
    gain = 1 + 0.1 * rnd((K,), torch.float32, 86)
    positions = torch.tensor(random.Random(87).choices(range(max_ctx), k=M), dtype=torch.int32)
    slots = torch.tensor(random.Random(88).sample(range(n_pages * page_size), M), dtype=torch.int32)
    plane0 = rnd((n_pages, 2, n_kv, page_size, hd), dtype, 89)
    pa, pb = plane0.clone().cuda(), plane0.clone()
    got = ops.qkv_rope(x.cuda(), w.cuda(), (gain.cuda(), 1e-5), positions.cuda(), slots.cuda(), table.cuda(), pa, n_heads,
                       n_kv, hd, page_size, interleaved).cpu()
    want = ref.qkv_rope(x, w, (gain, 1e-5), positions, slots, table, pb, n_heads, n_kv, hd, page_size, interleaved)
    t = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    torch.testing.assert_close(got.float(), want.float(), **t)
    torch.testing.assert_close(pa.cpu().float(), pb.float(), **t)
    # against the formula itself: natural-order weights, rotate_half pairing (reference main_models_new.py:71-80)
    if not interleaved:
        half = hd // 2
        order = torch.stack((torch.arange(half), torch.arange(half) + half), dim=1).reshape(-1)
        inv = torch.argsort(order)
        wq = w[:n_heads * hd].view(n_heads, hd, K)[:, inv].reshape(n_heads * hd, K)      # back to natural order
        q = (ref.rmsnorm(x, gain, 1e-5).double() @ wq.double().t()).view(M, n_heads, hd)
        c, s = table[positions.long()][..., 0].double().repeat(1, 2).unsqueeze(1), table[positions.long()][..., 1].double().repeat(1, 2).unsqueeze(1)
        rot = torch.cat((-q[..., half:], q[..., :half]), dim=-1)
        torch.testing.assert_close(got.double().view(M, n_heads, hd), q * c + rot * s, **t)


@pytest.mark.parametrize("first", [0, 60, 120])
def test_products_of_drawn_shapes(ops_for, first):
    """Sixty products a case with the rows (1 to 2,100), both widths (aligned to 16, 8, 4 or 2, or to nothing) and the
    kind (plain, with residual, with the norm in front, gated, 32-bit results) drawn at random: whichever kernel the
    route picks for a shape (few rows, tiles, or the plain one for unaligned operands), the result is the reference's."""
    ops, ref = ops_for(torch.bfloat16), TorchOps(dtype=torch.bfloat16)
    for case in range(first, first + 60):
        rng = random.Random(5000 + case)
        M = rng.choice([rng.randint(1, 8), rng.randint(9, 32), rng.randint(33, 128), rng.randint(129, 600), rng.randint(600, 2100)])
        N = rng.choice([rng.randint(1, 64) * 4, rng.randint(8, 300) * 8, rng.randint(100, 1100) * 8, rng.randint(1, 2000) * 2,
                        rng.randint(1, 3000)])
        K = rng.choice([rng.randint(1, 40) * 8, rng.randint(8, 560) * 8, rng.randint(8, 280) * 16, rng.randint(1, 500) * 2])
        kind = rng.choice(["plain", "residual", "norm", "norm+residual", "f32", "gate", "norm+gate"])
        if "gate" in kind:
            N = max(2, N // 2 * 2)
        x, w = rnd((M, K), torch.bfloat16, case * 3 + 1, 2.0), rnd((N, K), torch.bfloat16, case * 3 + 2, K ** -0.5)
        gain, res = 1 + 0.1 * rnd((K,), torch.float32, case * 3 + 3), rnd((M, N), torch.bfloat16, case * 3 + 4)
        rms_there, rms_here = ((gain.cuda(), 1e-5), (gain, 1e-5)) if "norm" in kind else (None, None)
        if "gate" in kind:
            got, want = ops.linear_swiglu(x.cuda(), w.cuda(), rms=rms_there), ref.linear_swiglu(x, w, rms=rms_here)
        elif kind == "f32":
            got, want = ops.linear(x.cuda(), w.cuda(), out_dtype=torch.float32), ref.linear(x, w, out_dtype=torch.float32)
        else:
            with_res = "residual" in kind
            got = ops.linear(x.cuda(), w.cuda(), residual=res.clone().cuda() if with_res else None, rms=rms_there)
            want = ref.linear(x, w, residual=res.clone() if with_res else None, rms=rms_here)
        torch.testing.assert_close(got.cpu().float(), want.float(), rtol=3e-2, atol=3e-2,
                                   msg=lambda m_: f"case {case}: {kind}, {M} rows, {N} out, {K} in: {m_}")


@pytest.mark.parametrize("M", [1, 8, 16, 20, 40, 70])
def test_skinny_product_with_two_column_tiles_a_workgroup(ops_for, M):
    """Very wide matrices give a workgroup of the staged kernel two column tiles. Forced here at a small width that
    ends inside the second tile, for the plain, the 32-bit and the normed and gated product, with one and with two
    blocks of 16 rows, and with two stages of LDS instead of four."""
    ops, ref = ops_for(torch.bfloat16), TorchOps(dtype=torch.bfloat16)
    N, K = 138, 800
    x, w = rnd((M, K), torch.bfloat16, 91, 2.0), rnd((N, K), torch.bfloat16, 92, K ** -0.5)
    gain = 1 + 0.1 * rnd((K,), torch.float32, 93)
    ops.gemm_skinny.cdll.tis_gemm_skinny_staged_always(1)
    try:
        narrow = [ops.linear(x.cuda(), w.cuda()).cpu(), ops.linear(x.cuda(), w.cuda(), out_dtype=torch.float32).cpu(),
                  ops.linear_swiglu(x.cuda(), w.cuda(), rms=(gain.cuda(), 1e-5)).cpu()]
        ops.gemm_skinny.cdll.tis_gemm_skinny_wide_tiles(1)
        wide = [ops.linear(x.cuda(), w.cuda()).cpu(), ops.linear(x.cuda(), w.cuda(), out_dtype=torch.float32).cpu(),
                ops.linear_swiglu(x.cuda(), w.cuda(), rms=(gain.cuda(), 1e-5)).cpu()]
        ops.gemm_skinny.cdll.tis_gemm_skinny_staged_stages(2)
        wide2 = [ops.linear(x.cuda(), w.cuda()).cpu(), ops.linear(x.cuda(), w.cuda(), out_dtype=torch.float32).cpu(),
                 ops.linear_swiglu(x.cuda(), w.cuda(), rms=(gain.cuda(), 1e-5)).cpu()]
    finally:
        ops.gemm_skinny.cdll.tis_gemm_skinny_wide_tiles(256)
        ops.gemm_skinny.cdll.tis_gemm_skinny_staged_stages(0)
        ops.gemm_skinny.cdll.tis_gemm_skinny_staged_always(0)
    for a, b, c in zip(narrow, wide, wide2):
        assert torch.equal(a, b)          # the same sums in the same order, only spread over workgroups differently
        assert torch.equal(a, c)
    torch.testing.assert_close(wide[1].double(), x.double() @ w.double().t(), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("V", [777, 48000])
def test_sampling_with_the_context_kept_on_the_device(sampling_kernel, V):
    """The penalty's context as a byte table per request instead of a token list: same draws, and the kernel marks
    what it drew."""
    ops = sampling_kernel
    n = 5
    logits = rnd((n, V), torch.float32, 90, 3.0)
    temperature = torch.tensor([0.0, 1.0, 0.8, 1.0, 0.9])
    top_k = torch.tensor([0, 40, 0, 3, 50], dtype=torch.int32)
    top_p = torch.tensor([0.0, 0.9, 0.0, 0.9, 0.95])
    pen = torch.tensor([1.5, 1.2, 1.0, 1.3, 1.1])
    ctx = [torch.tensor(sorted(set(random.Random(91 + i).choices(range(V), k=30))), dtype=torch.int32) for i in range(n)]
    off = torch.tensor([0] + list(torch.tensor([len(c) for c in ctx]).cumsum(0)), dtype=torch.int32)
    u = torch.rand(n, generator=torch.Generator().manual_seed(92))
    by_list = ops.sample(logits.cuda(), temperature.cuda(), top_k.cuda(), top_p.cuda(), pen.cuda(), u.cuda(),
                         torch.cat(ctx).cuda(), off.cuda()).cpu()
    seen = torch.zeros(8, V, dtype=torch.uint8)
    lines = torch.tensor([6, 0, -1, 3, 2], dtype=torch.int32)          # row 2 has no penalty and no line
    for i in range(n):
        if lines[i] >= 0:
            seen[lines[i], ctx[i].long()] = 1
    seen_gpu = seen.cuda()
    by_table = ops.sample(logits.cuda(), temperature.cuda(), top_k.cuda(), top_p.cuda(), pen.cuda(), u.cuda(),
                          seen=seen_gpu, seen_row=lines.cuda()).cpu()
    assert by_table.tolist() == by_list.tolist()
    after = seen_gpu.cpu()
    for i in range(n):
        if lines[i] >= 0:
            want = seen[lines[i]].clone(); want[by_table[i]] = 1
            assert torch.equal(after[lines[i]], want)
    assert torch.equal(after[[1, 4, 5, 7]], seen[[1, 4, 5, 7]])


def test_the_measurement_tool_runs(capsys):
    """python -m tiny_inference_server_amd.ops.kernel_bench, the tool that the counter profiles under profiles/ were
    made with: one small case of each kind runs and prints its line."""
    from tiny_inference_server_amd.ops.kernel_bench import main
    assert main(["attention", "--segments", "100:1x3,0:40", "--heads", "4", "--kv-heads", "2", "--head-dim", "64", "--reps", "2"]) == 0
    assert main(["product", "--rows", "8", "--out", "96", "--in", "64", "--kind", "norm+gate", "--reps", "2"]) == 0
    assert main(["product", "--rows", "40", "--out", "96", "--in", "64", "--kind", "residual", "--copies", "3", "--reps", "2"]) == 0
    out = capsys.readouterr().out
    assert out.count(" us; ") == 3 and "attention 100:1x3,0:40" in out and "product residual rows 40" in out
