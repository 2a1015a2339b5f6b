"""Host-side check of the index arithmetic behind the dropout debug keep-mask stores of the forward tile kernel
(torch_mlu_amd/csrc/fa_fwd_kernels.hip: `drow`, `row_in`, `col_lim`): for packed sequences that are longer than the
`max_seqlen_q` / `max_seqlen_k` the caller stated — the case in which the unclamped arithmetic left the tensor — every
store the guards let through lies inside the [seqlen_q, seqlen_k] plane of its own (sequence, head).  The GPU test of
the same case is tests/test_gpu_dropout.py::test_debug_mask_of_a_sequence_longer_than_stated_stays_inside_its_plane;
this one runs the arithmetic alone, over many random shapes, without a GPU."""
import numpy as np
import pytest

BM, BN = 128, 64


def _stores(batch, heads, seqlen_q, seqlen_k, lens_q, lens_k, causal, top_left):
    """All (byte offset, byte count) the kernel's guards admit, for every (sequence, head, row, column pair)."""
    out = []
    for b in range(batch):
        Lq, Lk = lens_q[b], lens_k[b]
        if Lq <= 0:
            continue
        off = 0 if top_left else Lk - Lq
        nblk = (Lq + BM - 1) // BM
        rows = np.arange(nblk * BM)                                # every row a wavefront lane may own
        ntiles = (Lk + BN - 1) // BN
        cols = np.arange(0, ntiles * BN, 2)                        # first column of every pair a lane may own
        r, c = np.meshgrid(rows, cols, indexing="ij")
        last_k = Lk - 1
        causal_row_lim = r + off if causal else np.full_like(r, 0x7fffffff)
        row_in = (r < Lq) & (r < seqlen_q)
        col_lim = np.minimum(np.minimum(last_k, causal_row_lim), seqlen_k - 1)
        pair = row_in & (c + 1 <= col_lim)
        single = row_in & ~pair & (c <= col_lim)
        row_clamped = np.minimum(r, min(Lq, seqlen_q) - 1)
        for h in range(heads):
            plane = (b * heads + h) * seqlen_q
            base = (plane + row_clamped) * seqlen_k * 2 + c * 2
            out.append((b, h, base[pair], 4))
            out.append((b, h, base[single], 2))
    return out


@pytest.mark.parametrize("seed", range(40))
def test_debug_mask_stores_stay_inside_their_plane(seed):
    rng = np.random.default_rng(seed)
    batch, heads = int(rng.integers(1, 4)), int(rng.integers(1, 3))
    seqlen_q, seqlen_k = int(rng.integers(1, 200)), int(rng.integers(1, 300))
    # some sequences are longer than stated, some shorter, some empty
    lens_q = [int(rng.integers(0, 2 * seqlen_q + 2)) for _ in range(batch)]
    lens_k = [int(rng.integers(0, 2 * seqlen_k + 2)) for _ in range(batch)]
    causal, top_left = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    total = batch * heads * seqlen_q * seqlen_k * 2
    n = 0
    for b, h, offs, size in _stores(batch, heads, seqlen_q, seqlen_k, lens_q, lens_k, causal, top_left):
        if offs.size == 0:
            continue
        lo = (b * heads + h) * seqlen_q * seqlen_k * 2
        hi = lo + seqlen_q * seqlen_k * 2
        assert offs.min() >= lo and offs.max() + size <= hi <= total
        # a store never crosses the end of its row either (the next row belongs to another query)
        assert np.all((offs - lo) % (seqlen_k * 2) + size <= seqlen_k * 2)
        n += offs.size
    if any(l > 0 for l in lens_q) and any(l > 0 for l in lens_k) and not causal:
        assert n > 0


def test_the_unclamped_arithmetic_is_what_left_the_plane():
    """The same walk with the guards the kernel used to have (row < Lq, col <= last_k only) does leave the plane when a
    sequence is longer than stated: the check above is not vacuous."""
    seqlen_q, seqlen_k, Lq, Lk = 64, 96, 100, 150
    r, c = np.meshgrid(np.arange(BM), np.arange(0, ((Lk + BN - 1) // BN) * BN, 2), indexing="ij")
    admitted = (r < Lq) & (c <= Lk - 1)
    offs = (np.minimum(r, Lq - 1) * seqlen_k + c)[admitted] * 2
    assert offs.max() >= seqlen_q * seqlen_k * 2
