"""The oracle's weight pre-shuffle (the MI355X counterpart of construct_m16n8k32_B_layout,
src/base/base.cu:222-271), pinned without the GPU by what the layout is for:

* it is a permutation of 16-byte chunks that keeps every chunk inside its own 2 KB block
  (16 rows x one 128-K slice) and inside its own row's 128-byte line of that block, and the
  inverse restores the input exactly (the reference checks its permutation by exact inversion,
  examples/005.fp8.mm.opt.cu:710-765);
* the MFMA operand read of the image -- lane (g, i) takes row i, chunks 2g and 2g+1 -- finds the
  bytes k = 32g .. 32g+31 of row i, and every quarter-wave pass of a 16-byte LDS read touches 16
  different 16-byte slots of the 256-byte bank row (no bank conflict);
* a wave's linear 1 KB copy (lane l moves bytes 16l .. 16l+15 of a half block) covers whole rows.
"""
import numpy as np
import pytest


def _chunk_ids(N, K):
    """A byte matrix whose 16-byte chunks carry their own (row, chunk) identity."""
    ids = np.arange(N * (K // 16), dtype=np.uint64).reshape(N, K // 16)
    out = np.zeros((N, K // 16, 16), np.uint8)
    for b in range(8):
        out[:, :, b] = (ids >> np.uint64(8 * b)).astype(np.uint8)
    out[:, :, 8:] = np.arange(8, dtype=np.uint8) + 1  # position inside the chunk
    return out.reshape(N, K), ids


@pytest.mark.parametrize("N,K", [(16, 128), (48, 384), (128, 256), (256, 1280)])
def test_permutation_of_chunks_confined_to_block_and_row(oracle, N, K):
    x, ids = _chunk_ids(N, K)
    p = oracle.preshuffle_b(x)
    assert p.shape == x.shape and p.dtype == np.uint8
    chunks = p.reshape(-1, 16)
    assert (chunks[:, 8:] == np.arange(8, dtype=np.uint8) + 1).all(), "bytes moved inside a chunk"
    got = np.zeros(chunks.shape[0], np.uint64)
    for b in range(8):
        got |= chunks[:, b].astype(np.uint64) << np.uint64(8 * b)
    assert np.array_equal(np.sort(got), np.arange(N * K // 16, dtype=np.uint64)), "not a permutation of the chunks"
    row, chunk = got // np.uint64(K // 16), got % np.uint64(K // 16)
    pos = np.arange(got.size)
    blk, within = pos // 128, pos % 128  # 128 chunks per 2 KB block
    assert np.array_equal(blk, (row // 16) * (K // 128) + chunk // 8), "a chunk left its (16 rows x 128 K) block"
    assert np.array_equal(within // 8, row % 16), "a chunk left its row's 128-byte line"
    assert np.array_equal(oracle.unshuffle_b(p), x)
    assert np.array_equal(oracle.preshuffle_b(oracle.unshuffle_b(x)), x)


def test_operand_reads_find_their_bytes_and_do_not_conflict(oracle):
    rng = np.random.default_rng(5)
    x = rng.integers(0, 256, (16, 128), dtype=np.uint8)
    img = oracle.preshuffle_b(x).reshape(-1)
    swz = oracle.operand_swizzle_rows16(np.arange(16))
    # quarter-wave passes of a 16-byte LDS read on gfx950 (lanes served together)
    first = [0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27]
    second = [4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31]
    passes = [first, second, [l + 32 for l in first], [l + 32 for l in second]]
    for half in (0, 1):  # the two 16-byte reads of a lane: chunk 2g, then 2g + 1
        offs = {}
        for lane in range(64):
            g, i = lane // 16, lane % 16
            off = i * 128 + (((2 * g + half) ^ int(swz[i])) << 4)
            offs[lane] = off
            assert np.array_equal(img[off:off + 16], x[i, 32 * g + 16 * half:32 * g + 16 * half + 16])
        for lanes in passes:
            slots = {(offs[l] >> 4) & 15 for l in lanes}
            assert len(slots) == 16, "bank conflict in an operand read pass"
    # second read = first read with address bit 4 flipped (what the kernels rely on)
    for i in range(16):
        for g in range(4):
            a0 = i * 128 + (((2 * g) ^ int(swz[i])) << 4)
            a1 = i * 128 + (((2 * g + 1) ^ int(swz[i])) << 4)
            assert a1 == a0 ^ 16


def test_linear_kilobyte_copy_covers_whole_rows(oracle):
    x, ids = _chunk_ids(16, 128)
    chunks = oracle.preshuffle_b(x).reshape(-1, 16)
    got = np.zeros(chunks.shape[0], np.uint64)
    for b in range(8):
        got |= chunks[:, b].astype(np.uint64) << np.uint64(8 * b)
    for half in (0, 1):
        rows = (got[64 * half:64 * half + 64] // np.uint64(8)).astype(int)
        assert sorted(set(rows.tolist())) == list(range(8 * half, 8 * half + 8))
        assert all((rows == r).sum() == 8 for r in range(8 * half, 8 * half + 8))


def test_alignment_errors_carry_the_reference_texts(oracle):
    with pytest.raises(RuntimeError, match="K must be greater than 0 and divisible by 128."):
        oracle.preshuffle_b(np.zeros((16, 100), np.uint8))
    with pytest.raises(RuntimeError, match="M or N can't be divided 128."):
        oracle.transpose_aligned_128(np.zeros((128, 100), np.uint8))
