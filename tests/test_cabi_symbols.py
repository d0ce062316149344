"""The built C-ABI library loads on a machine without a GPU and exports exactly the entry
points include/syncopate_hip.h declares; host-only entry points behave as documented."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "syncopate_hip.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(syn_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from syncopate_amd import _lib

    if not _lib.LIB_PATH.exists():
        from syncopate_amd.build import build_library

        build_library(verbose=False)
    return _lib.load()


def test_header_and_library_agree(lib):
    from syncopate_amd import _lib

    declared = _declared()
    assert declared == sorted(_lib.EXPORTED_SYMBOLS)
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.syn_version() >= 100


def test_constants_match_the_header():
    """Every numeric SYN_* constant the Python binding mirrors has the header's value, and every option
    bit of the header is mirrored (a launcher that set a stale bit would silently run another form)."""
    from syncopate_amd import _lib

    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    header = {name: int(value.rstrip("uU"), 0)
              for name, value in re.findall(r"#define\s+(SYN_[A-Z0-9_]+)\s+\(?(-?(?:0x[0-9a-fA-F]+|\d+)[uU]?)\)?\s*$", text, flags=re.M)}
    assert len(header) > 20
    mirrored = {name: getattr(_lib, name) for name in header if hasattr(_lib, name)}
    assert mirrored == {name: header[name] for name in mirrored}
    for name in header:
        if name.startswith(("SYN_GEMM_", "SYN_ATTN_", "SYN_E")):
            assert name in mirrored, name


def test_struct_layouts_match_the_header():
    """Field order and count of the ctypes mirrors follow the header's structs."""
    from syncopate_amd import _lib

    text = open(HEADER).read()
    for struct, mirror in (("syn_gemm_desc", _lib.GemmDesc), ("syn_attn_desc", _lib.AttnDesc)):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (struct, struct), text, flags=re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        names = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            for part in decl.split(","):
                names.append(re.findall(r"[A-Za-z_][A-Za-z0-9_]*", part)[-1])
        assert names == [f[0] for f in mirror._fields_], struct


def test_gemm_wave_check_host_only(lib):
    from syncopate_amd import _lib

    def check(sizes, offsets, signals, M=512, N=256, K=128, bm=128, bn=128, cum=512 * 256, flags=4):
        n = len(signals)
        s = (ctypes.c_int32 * (2 * n))(*[x for row in sizes for x in row])
        o = (ctypes.c_int32 * (2 * n))(*[x for row in offsets for x in row])
        g = (ctypes.c_int32 * n)(*signals)
        return lib.syn_gemm_check_waves(s, o, g, n, M, N, K, bm, bn, 64, cum, flags)

    good = ([[256, 256], [256, 256]], [[256, 0], [0, 0]], [-1, 0])
    assert check(*good) == 0
    assert check([[256, 256], [256, 256]], [[0, 0], [512, 0]], [-1, 0]) == _lib.SYN_ERANGE
    assert check(*good[:2], [-1, 4]) == _lib.SYN_ERANGE
    assert check(*good[:2], [-1, -2]) == _lib.SYN_EINVAL
    assert check([[256, 256], [200, 256]], good[1], good[2]) == _lib.SYN_EINVAL
    assert check([[256, 256]], [[0, 0]], [-1]) == _lib.SYN_EINVAL            # does not add up to cum_tiles
    assert check(*good, K=100) == _lib.SYN_EINVAL
    assert lib.syn_gemm_grid(8192 * 3584, 8192, 3584, 128, 256, 256) == 256
    assert lib.syn_gemm_grid(0, 256, 256, 128, 128, 256) == 4
    assert lib.syn_gemm_grid(0, 256, 256, 0, 128, 256) == _lib.SYN_EINVAL


def test_attn_wave_check_host_only(lib):
    from syncopate_amd import _lib

    def check(offsets, sizes, cums, signals, Z=1, H=2, Sq=256, Skv=512, cum=None, flags=2):
        n = len(cums)
        o = (ctypes.c_int32 * (4 * n))(*[x for row in offsets for x in row])
        s = (ctypes.c_int32 * (4 * n))(*[x for row in sizes for x in row])
        c = (ctypes.c_int32 * n)(*cums)
        g = (ctypes.c_int32 * n)(*signals)
        return lib.syn_attn_check_waves(o, s, c, g, n, Z, H, Sq, Skv, 128, 128,
                                        cums[-1] if cum is None else cum, flags)

    offsets, sizes = [[0, 0, 0, 256], [0, 0, 0, 0]], [[1, 2, 256, 256]] * 2
    assert check(offsets, sizes, [512, 1024], [-1, 0]) == 0
    assert check(offsets, sizes, [512, 1000], [-1, 0]) == _lib.SYN_EINVAL      # prefix sum is wrong
    assert check([[0, 0, 0, 384], [0, 0, 0, 0]], sizes, [512, 1024], [-1, 0]) == _lib.SYN_ERANGE
    assert check(offsets, sizes, [512, 1024], [-1, 2]) == _lib.SYN_ERANGE
    # zero-filled padding rows after the real waves are allowed
    assert check(offsets + [[0] * 4] * 2, sizes + [[0] * 4] * 2, [512, 1024, 0, 0], [-1, 0, 0, 0], cum=1024) == 0
    assert check([[0] * 4] + offsets, [[0] * 4] + sizes, [0, 512, 1024], [0, -1, 0], cum=1024) == _lib.SYN_EINVAL


def test_launch_entry_points_reject_null_descriptors_without_a_gpu(lib):
    from syncopate_amd import _lib

    assert lib.syn_gemm_consumer(None, None) == _lib.SYN_EINVAL
    assert lib.syn_attn_fwd(None, None) == _lib.SYN_EINVAL
    assert lib.syn_ring_reduce(None, None, None, 8, 0, 16, 16, 0, 0, None) == _lib.SYN_EINVAL
    assert lib.syn_flag_set(None, 1, None) == _lib.SYN_EINVAL
    assert lib.syn_delay_us(-1, None) == _lib.SYN_EINVAL
    desc = _lib.GemmDesc()
    assert lib.syn_gemm_consumer(ctypes.byref(desc), None) == _lib.SYN_EINVAL
