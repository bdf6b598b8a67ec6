"""Host logic of the dense launch plan, through the one function of it the library exports for sizing
a workspace: the bytes of split-K scratch, = tiles x K split x tile rows x 256 columns x 4.  No GPU call
is made (the plan is arithmetic on the shape)."""
import ctypes as C

import pytest

from rknpu2_matmul_open_amd import capi


@pytest.fixture(scope="module")
def scratch_bytes():
    lib = capi.load_library()
    f = lib.rkh_gemm_scratch_bytes
    f.restype = C.c_size_t
    f.argtypes = [C.c_int] * 4
    return f


def _ksplit(nbytes, M, N):
    """K split implied by the scratch size (rows are padded to the tile, so try every tile height)."""
    found = set()
    for bm in (128, 64, 32):
        tiles = -(-M // bm) * -(-N // 256)
        per_part = tiles * bm * 256 * 4
        if nbytes % per_part == 0:
            found.add(nbytes // per_part)
    return found


# (M, N, K, int4) -> K split the plan chooses; the choices measured fastest (or within a few percent of it)
# among forced plans on the device: long K with few columns is split, wide or short-K GEMMs are not
PINNED = [((192, 4096, 4096, 0), 4), ((256, 4096, 4096, 0), 4), ((512, 4096, 4096, 0), 0), ((1024, 4096, 4096, 0), 0),
          ((192, 11008, 4096, 0), 0), ((512, 11008, 4096, 0), 0), ((1024, 14336, 4096, 0), 0),
          ((192, 4096, 11008, 0), 4), ((256, 4096, 11008, 0), 4), ((512, 4096, 11008, 0), 4), ((1024, 4096, 11008, 0), 2),
          ((2048, 4096, 4096, 1), 0), ((2048, 4096, 4096, 0), 0), ((512, 4096, 11008, 1), 2), ((192, 4096, 4096, 1), 0)]


@pytest.mark.parametrize("shape,ksplit", PINNED)
def test_k_split_of_measured_shapes(scratch_bytes, shape, ksplit):
    M, N, K, int4 = shape
    nbytes = scratch_bytes(M, N, K, int4)
    if ksplit == 0:
        assert nbytes == 0
    else:
        assert ksplit in _ksplit(nbytes, M, N), (nbytes, _ksplit(nbytes, M, N))


def test_plan_invariants(scratch_bytes):
    # decode-sized calls never split over workgroups
    for M in range(1, 9):
        assert scratch_bytes(M, 4096, 14336, 0) == 0 and scratch_bytes(M, 4096, 14336, 1) == 0
    # int4 weights ride as 16 x code: a part may not span more than 2^17 k, whatever the estimate prefers
    for M in (200, 2000):
        nbytes = scratch_bytes(M, 96, 131072 + 2112, 1)
        assert nbytes > 0 and min(_ksplit(nbytes, M, 96)) >= 2
        nbytes = scratch_bytes(M, 96, 3 * 131072 + 64, 1)
        assert nbytes > 0 and min(_ksplit(nbytes, M, 96)) >= 4
    # a part keeps at least 1024 k, and the scratch stays bounded
    assert scratch_bytes(4000, 256, 1500, 0) == 0
    for shape in ((300001, 300, 33, 0), (100000, 256, 8192, 0), (5000, 64, 60000, 0), (129, 3000001, 40, 0)):
        assert scratch_bytes(*shape) <= 512 * 1000 * 1000


def test_which_moe_calls_take_the_two_launch_path():
    """Up to twelve tokens, a hidden size that fits the staging area, a middle short enough for nine
    re-quantized rows side by side; everything else takes the routed, grouped path."""
    lib = capi.load_library()
    f = lib.rkh_moe_decode_applies
    f.restype = C.c_int
    f.argtypes = [C.c_int] * 3
    for rows in range(1, 13):
        assert f(rows, 2048, 1024) and f(rows, 64, 32) and f(rows, 32768, 3584)
    assert not f(13, 2048, 1024) and not f(256, 2048, 1024) and not f(0, 2048, 1024)
    assert not f(4, 32768 + 32, 1024) and not f(4, 2048, 3584 + 32) and not f(4, 2048, 8192)
    assert not f(4, 2040, 1024) and not f(4, 2048, 1000)   # (the layer's geometry is in multiples of 32)
