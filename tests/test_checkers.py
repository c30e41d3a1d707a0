"""CPU: the checkers of the full-size GPU parity tests catch what they are there to catch.

A product that is right everywhere except in one 32x32 block of C (a border tile that dropped its last
k-slab, a wavefront's block written to the wrong rows) must fail the entry-by-entry comparison and the
lattice; an error in a single entry must fail the entry-by-entry comparison."""
import numpy as np
import pytest

from helpers import (assert_every_entry, gemm_bound_fast, gemm_errors_everywhere, lattice_errors,
                     lattice_points)
from wekua_amd import synth


def _case(M=320, N=288, K=256):
    a = synth.uniform(71, (M, K), np.float32)
    b = synth.uniform(72, (K, N), np.float32)
    c = synth.uniform(73, (M, N), np.float32)
    want = (1.5 * (a.astype(np.float64) @ b.astype(np.float64)) + 0.5 * c).astype(np.float32)
    bound = gemm_bound_fast("f32", 1.5, a, 0, b, 0, 0.5, c)
    return a, b, c, want, bound, K


def test_a_correct_product_passes():
    a, b, c, want, bound, K = _case()
    assert_every_entry("f32", want.copy(), want, bound, K)
    ii, jj, err = lattice_errors("f32", want, 1.5, a, 0, b, 0, 0.5, c, K)
    assert err.max() <= 1.0


@pytest.mark.parametrize("block", [(0, 0), (3, 5), (9, 8)])
def test_one_block_without_its_last_k_slab_is_caught(block):
    a, b, c, want, bound, K = _case()
    bi, bj = block
    rows, cols = slice(32 * bi, 32 * bi + 32), slice(32 * bj, 32 * bj + 32)
    got = want.copy()
    got[rows, cols] = (1.5 * (a[rows, :K - 16].astype(np.float64) @ b[:K - 16, cols].astype(np.float64)) + 0.5 * c[rows, cols])
    with pytest.raises(AssertionError, match="beyond the tolerance"):
        assert_every_entry("f32", got, want, bound, K)
    ii, jj, err = lattice_errors("f32", got, 1.5, a, 0, b, 0, 0.5, c, K)
    bad = err > 1.0
    assert bad.any()
    inside = (ii[bad] // 32 == bi) & (jj[bad] // 32 == bj)
    assert inside.all()


def test_two_blocks_swapped_are_caught():
    a, b, c, want, bound, K = _case()
    got = want.copy()
    got[32:64, 0:32], got[64:96, 0:32] = want[64:96, 0:32], want[32:64, 0:32]
    with pytest.raises(AssertionError):
        assert_every_entry("f32", got, want, bound, K)
    _, _, err = lattice_errors("f32", got, 1.5, a, 0, b, 0, 0.5, c, K)
    assert err.max() > 1.0


def test_a_single_wrong_entry_is_caught_by_the_whole_comparison():
    a, b, c, want, bound, K = _case()
    got = want.copy()
    got[201, 77] += 0.5
    err = gemm_errors_everywhere("f32", got, want, bound, K)
    assert (err > 1.0).sum() == 1
    with pytest.raises(AssertionError, match=r"\(201, 77\)"):
        assert_every_entry("f32", got, want, bound, K)


@pytest.mark.parametrize("shape", [(8192, 8192), (4097, 4095), (8192, 256), (1000, 1000)])
def test_the_lattice_visits_every_block_and_every_position_of_a_block(shape):
    M, N = shape
    ii, jj = lattice_points(M, N, ragged_edges=False)
    blocks = set(zip((ii // 32).tolist(), (jj // 32).tolist()))
    assert len(blocks) == ((M + 31) // 32) * ((N + 31) // 32)
    if M % 32 == 0 and N % 32 == 0 and len(blocks) >= 4096:
        slots = set(((ii % 32) * 32 + jj % 32).tolist())
        assert len(slots) == 1024          # 64 lanes x 16 accumulator registers of a 32x32 block
    ii, jj = lattice_points(M, N)
    pts = set(zip(ii.tolist(), jj.tolist()))
    assert all((M - 1, j) in pts for j in range(N)) and all((i, N - 1) in pts for i in range(M))
