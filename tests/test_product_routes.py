"""Which kernel a bfloat16 matrix product goes to, checked on the host with recording stand-ins for the compiled
libraries: the library's product only ever sees widths from its list, at row counts of one family, with a result that
is not the residual and operands whose memory reaches as far as the rows it is asked for."""
from __future__ import annotations

import random
from ctypes import c_void_p

import pytest
import torch

from tiny_inference_server_amd.ops import hip_ops
from tiny_inference_server_amd.ops.hip_ops import HipOps, KernelError, library_rows, library_widths, product_route


class Recorder:
    """Stands in for a compiled library: every entry point records its arguments and does nothing."""

    def __init__(self, calls, name):
        self._calls, self._name = calls, name

    def __getattr__(self, fn):
        def call(*args):
            self._calls.append((fn, [(a.value or 0) if isinstance(a, c_void_p) else a for a in args]))
        return call


def host_ops(widths=None, few_rows=hip_ops._FEW_ROWS):
    """The operations object without a device: its dispatch is real, its libraries record."""
    ops = object.__new__(HipOps)
    ops.device = torch.device("cpu")
    ops._device_index = 0
    ops.dtype, ops.code = torch.bfloat16, 1
    ops.few_rows = few_rows
    ops.library_widths = library_widths() if widths is None else frozenset(widths)
    ops._warned_widths = set()
    ops.calls = []
    for lib in ("rowwise", "gemm_skinny", "gemm_library", "gemm_plain", "gemm_tiles"):
        setattr(ops, lib, Recorder(ops.calls, lib))
    ops._stream = lambda: c_void_p(0)
    return ops


def inside(t, ptr, rows, ld, width):
    """Whether `rows` rows of `width` elements at stride `ld` from `ptr` lie in the memory behind tensor t."""
    base = t.untyped_storage().data_ptr()
    end = base + t.untyped_storage().nbytes()
    return base <= ptr and ptr + ((rows - 1) * ld + width) * t.element_size() <= end


def test_library_rows_family():
    assert [library_rows(m) for m in (1, 33, 64, 65, 72, 128, 200, 256)] == [64, 64, 64, 128, 128, 128, 256, 256]
    assert [library_rows(m) for m in (257, 2022, 2046, 2047, 2048, 2056, 2112, 4097)] == \
        [512, 2048, 2048, 2048, 2048, 2304, 2304, 4352]
    for m in range(1, 5000, 7):
        r = library_rows(m)
        assert r >= m and r % 64 == 0 and (r <= 256 or r % 256 == 0) and r - m < 256


def test_routes():
    w = {(2304, 1536)}
    assert product_route(8, 2304, 1536, True, False, w) == "few_rows"
    assert product_route(64, 2304, 1536, True, False, w, few_rows=64) == "few_rows"
    assert product_route(65, 2304, 1536, True, False, w, few_rows=64) == "library"
    assert product_route(hip_ops._FEW_ROWS, 2304, 1536, True, False, w) == "few_rows"
    assert product_route(hip_ops._FEW_ROWS + 1, 2304, 1536, True, False, w) == "library"
    assert product_route(2048, 2304, 1536, True, True, w) == "tiles"            # 32-bit results: own kernels
    assert product_route(100, 2304, 1536, True, True, w) == "few_rows"
    assert product_route(2048, 6144, 4096, True, False, w) == "tiles"           # a width nobody listed: own kernel
    assert product_route(128, 6144, 4096, True, False, w) == "few_rows"
    assert product_route(2048, 6146, 4096, True, False, w) == "few_rows"        # ... whose stores need N in steps of 4
    assert product_route(2048, 2304, 1536, False, False, w) == "plain"


def test_the_list_holds_no_width_of_the_largest_size():
    from tiny_inference_server_amd.__main__ import size_config
    cfg = size_config("7B")
    D, F = cfg.d_model, cfg.ffn_hidden
    qkv = (cfg.n_heads + 2 * cfg.n_kv_heads) * cfg.head_dim
    listed = library_widths()
    for pair in ((qkv, D), (D, D), (2 * F, D), (D, F), (cfg.vocab_size, D), (D, 2 * D)):
        assert pair not in listed, pair


@pytest.mark.parametrize("seed", range(4))
def test_no_unlisted_width_and_no_unrounded_row_count_reaches_the_library(seed):
    rng = random.Random(seed)
    listed = sorted(library_widths())
    ops = host_ops()
    held = []
    for _ in range(60):
        if rng.random() < 0.6:
            N, K = rng.choice(listed)
        else:
            N, K = rng.choice((6144, 4096, 28672, 96, 1000, 520)), rng.choice((4096, 14336, 64, 200, 1528))
        M = rng.choice((1, 8, 33, 64, 65, 72, 200, 257, 2022, 2047, 2048, 2056, 2112, rng.randrange(1, 4200)))
        if rng.random() < 0.5:
            x = ops.empty(M, K)                    # as the engine makes its activations
        else:
            x = torch.empty(M, K, dtype=torch.bfloat16)          # as a caller from outside would
        w = torch.empty(N, K, dtype=torch.bfloat16)
        res = ops.empty(M, N) if rng.random() < 0.5 else None
        n0 = len(ops.calls)
        out = ops.linear(x, w, residual=res, reuse_residual=bool(res is not None and rng.random() < 0.5),
                         rms=(torch.ones(K), 1e-5) if rng.random() < 0.3 else None)
        held.append((x, w, res, out))
        assert out.shape == (M, N)
        products = [c for c in ops.calls[n0:] if c[0].startswith("tis_gemm")]
        assert len(products) == 1
        fn, a = products[0]
        if fn == "tis_gemm_library":
            X, x_ld, W, R, r_ld, C, c_ld, rows, n, k, f32 = a[:11]
            assert (n, k) == (N, K) and (N, K) in library_widths() and M > ops.few_rows
            assert rows == library_rows(M) and f32 == 0
            assert C != R and (R != 0) == (res is not None)
            assert C == out.data_ptr() and inside(out, C, rows, c_ld, N)
            # the operands reach as far as the rows asked for, in memory that is theirs
            assert X % 16 == 0 and W % 16 == 0 and C % 16 == 0 and R % 16 == 0
            assert x_ld >= K and c_ld >= N
        elif fn == "tis_gemm_tiles":
            X, x_ld, W, R, r_ld, C, c_ld, rows, n, k, f32 = a[:11]
            assert (rows, n, k) == (M, N, K) and (N, K) not in library_widths() and M > ops.few_rows and f32 == 0
            assert K % 8 == 0 and N % 4 == 0 and X % 16 == 0 and W % 16 == 0 and C % 8 == 0 and R % 8 == 0
            assert C == out.data_ptr() and inside(out, C, M, c_ld, N) and x_ld >= K
        else:
            assert fn == "tis_gemm_skinny", fn
            assert M <= ops.few_rows or ((N, K) not in library_widths() and N % 4)


def test_rows_beyond_a_callers_tensor_are_never_read():
    """A tensor from outside has no memory behind its last row: the product runs on a copy that has."""
    ops = host_ops()
    N, K = sorted(library_widths())[0]
    M = 170
    x = torch.empty(M, K, dtype=torch.bfloat16)
    res = torch.empty(M, N, dtype=torch.bfloat16)
    ops.linear(x, torch.empty(N, K, dtype=torch.bfloat16), residual=res)
    fn, a = [c for c in ops.calls if c[0] == "tis_gemm_library"][0]
    assert a[7] == 192
    assert a[0] != x.data_ptr() and a[3] != res.data_ptr()
    # and one made by the operations object is used where it lies
    ops.calls.clear()
    x2, res2 = ops.empty(M, K), ops.empty(M, N)
    ops.linear(x2, torch.empty(N, K, dtype=torch.bfloat16), residual=res2)
    fn, a = [c for c in ops.calls if c[0] == "tis_gemm_library"][0]
    assert a[0] == x2.data_ptr() and a[3] == res2.data_ptr() and HipOps._holds_rows(x2, 192)


def test_unaligned_operands_go_to_the_plain_kernel():
    ops = host_ops()
    x = torch.empty(300, 1544, dtype=torch.bfloat16)[:, 3:1539]      # rows start 6 bytes into a 16-byte piece
    ops.linear(x, torch.empty(2304, 1536, dtype=torch.bfloat16))
    assert [c[0] for c in ops.calls if c[0].startswith("tis_gemm")] == ["tis_gemm_plain"]


def test_the_library_path_refuses_an_unlisted_width_even_if_asked_directly():
    ops = host_ops()
    with pytest.raises(KernelError, match="not among"):
        ops._linear_library(ops.empty(256, 4096), torch.empty(6144, 4096, dtype=torch.bfloat16), None)


def test_gated_and_projection_products_follow_the_same_routes():
    ops = host_ops()
    x = ops.empty(2112, 1536)
    ops.linear_swiglu(x, torch.empty(8192, 1536, dtype=torch.bfloat16), rms=(torch.ones(1536), 1e-5))
    kinds = [c[0] for c in ops.calls]
    assert kinds == ["tis_rmsnorm", "tis_gemm_library", "tis_swiglu"]
    assert [c for c in ops.calls if c[0] == "tis_gemm_library"][0][1][7] == 2304
    ops.calls.clear()
    ops.linear_swiglu(ops.empty(2112, 4096), torch.empty(28672, 4096, dtype=torch.bfloat16), rms=(torch.ones(4096), 1e-5))
    assert [c[0] for c in ops.calls] == ["tis_rmsnorm", "tis_gemm_tiles", "tis_swiglu"]    # an unlisted width: own tiles
    ops.calls.clear()
    ops.linear_swiglu(ops.empty(100, 4096), torch.empty(28672, 4096, dtype=torch.bfloat16), rms=(torch.ones(4096), 1e-5))
    assert [c[0] for c in ops.calls] == ["tis_gemm_skinny"]           # few rows: norm and gate fused
    assert hip_ops._FEW_ROWS == ops.few_rows
