"""The workgroup-id -> role map of the fused launch is a bijection: over a grid of GEMM tile counts, SpMM
block counts and group sizes, every tile and every block is the role of exactly one workgroup id.
Runs on the host (the device code calls the same function); no GPU."""
import ctypes

import pytest


def _roles(lib, G, S, g):
    ig, idx = ctypes.c_int(), ctypes.c_int()
    out = []
    for b in range(G + S):
        assert lib.iex_fused_role(G, S, g, b, ctypes.byref(ig), ctypes.byref(idx)) == 0
        out.append((ig.value, idx.value))
    return out


def test_every_tile_and_block_exactly_once():
    from intrasm_engine_amd import _lib
    lib = _lib.load()
    for G in list(range(0, 24)) + [59, 64, 100]:
        for S in list(range(0, 12)) + [39, 40, 257]:
            for g in (-1, -7, 0, 1, 2, 3, 4, 5, 7, 8, 11, 16, 64, 1000):
                roles = _roles(lib, G, S, g)
                assert sorted(i for is_gemm, i in roles if is_gemm) == list(range(G)), (G, S, g)
                assert sorted(i for is_gemm, i in roles if not is_gemm) == list(range(S)), (G, S, g)


def test_the_case_that_lost_tiles():
    """10 tiles, 1 block, groups of 4: an earlier map computed no role for tiles 3 and 7 and block -1."""
    from intrasm_engine_amd import _lib
    roles = _roles(_lib.load(), 10, 1, 4)
    assert roles == [(1, 0), (1, 1), (1, 2), (1, 3), (0, 0), (1, 4), (1, 5), (1, 6), (1, 7), (1, 8), (1, 9)]


def test_groups_keep_their_tiles_together_and_spread_the_blocks():
    from intrasm_engine_amd import _lib
    roles = _roles(_lib.load(), 8, 6, 4)      # two groups of 4 tiles, 3 blocks after each
    assert [r[0] for r in roles] == [1, 1, 1, 1, 0, 0, 0, 1, 1, 1, 1, 0, 0, 0]
    assert _roles(_lib.load(), 3, 2, 0) == [(1, 0), (1, 1), (1, 2), (0, 0), (0, 1)]
    # a negative group size: the blocks first (the longer jobs), then the tiles
    assert _roles(_lib.load(), 3, 2, -1) == [(0, 0), (0, 1), (1, 0), (1, 1), (1, 2)]


def test_arguments_are_checked():
    from intrasm_engine_amd import _lib
    lib = _lib.load()
    ig, idx = ctypes.c_int(), ctypes.c_int()
    assert lib.iex_fused_role(4, -4, 0, 0, ctypes.byref(ig), ctypes.byref(idx)) == -1
    assert lib.iex_fused_role(4, 4, 2, 8, ctypes.byref(ig), ctypes.byref(idx)) == -1
    assert "outside the grid" in _lib.last_error()
