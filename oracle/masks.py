"""CPU oracle: mask generators and the mask -> block-LUT compiler.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module;
it is the checker that tests, the smoke run and the CPU-baseline leg of the
bench compare the HIP path against.

Every function restates, in numpy with the same loop structure, one function of
the reference file ``src/util/masks.py`` (line ranges quoted per function).
The reference holds no golden vectors for this path, so the restatement is
pinned by closed forms, brute force and invariants (tests/test_oracle_masks.py):

* generators          - closed-form index predicates on every (i, j)
* get_sparse_storage  - exhaustive enumeration of all 2^16 masks on a 2x2 grid
                        of 2x2 blocks against an independent classifier, the
                        LUT -> dense round trip, and hand-derived block counts
* generate_bigbird_mask random part - restated call-for-call on the stdlib
                        Mersenne Twister; pinned additionally by a fixture the
                        reference generator itself produced
                        (tests/golden/bigbird_*.npz).
"""
import random

import numpy as np

NEG_MASK = -10000.0  # additive constant of a masked element, src/util/masks.py:160


def generate_causal_mask(attr_mask):
    """src/util/masks.py:10-14 - lower-triangular ones, repeated over batch."""
    b, s = attr_mask.shape[0], attr_mask.shape[1]
    tri = np.tril(np.ones((s, s), dtype=np.float32))
    return np.repeat(tri[None], b, axis=0)


def _causal_trim_last_batch(mask, batch):
    # The reference trims with the loop variable `batch` after the loop has
    # ended, i.e. only the LAST batch entry is made causal
    # (src/util/masks.py:28-30, 48-50, 77-79, 118-120).
    s = mask.shape[1]
    for i in range(s - 1):
        mask[batch, i, i + 1:] = 0


def generate_sliding_mask(attr_mask, bandwidth=1, is_cauasl=False):
    """src/util/masks.py:17-32 - |i-j| <= bandwidth."""
    b, s = attr_mask.shape[0], attr_mask.shape[1]
    m = np.zeros_like(attr_mask)
    batch = 0
    for batch in range(b):
        for i in range(s):
            m[batch, i, max(0, i - bandwidth):min(s, i + bandwidth + 1)] = 1
    if is_cauasl:
        _causal_trim_last_batch(m, batch)
    return m


def generate_dilated_mask(attr_mask, bandwidth=1, dilation_rate=1, is_cauasl=False):
    """src/util/masks.py:35-52 - columns i-bw-d, step d+1, up to i+bw+d, >= 0."""
    b, s = attr_mask.shape[0], attr_mask.shape[1]
    m = np.zeros_like(attr_mask)
    batch = 0
    for batch in range(b):
        for i in range(s):
            start = i - bandwidth - dilation_rate
            end = min(s, i + bandwidth + dilation_rate + 1)
            for col in range(start, end, dilation_rate + 1):
                if col > -1:
                    m[batch, i, col] = 1
    if is_cauasl:
        _causal_trim_last_batch(m, batch)
    return m


def generate_longformer_mask(attr_mask, globalwidth=1, bandwidth=1, is_cauasl=False):
    """src/util/masks.py:55-81 - global rows/cols at [0,g) and [S/2,S/2+g) + band."""
    b, s = attr_mask.shape[0], attr_mask.shape[1]
    m = np.zeros_like(attr_mask)
    batch = 0
    for batch in range(b):
        m[batch, :globalwidth, :] = 1
        m[batch, :, :globalwidth] = 1
    for batch in range(b):
        start = int(s / 2)
        end = int(s / 2 + globalwidth)
        m[batch, start:end, :] = 1
        m[batch, :, start:end] = 1
    for batch in range(b):
        for i in range(s):
            m[batch, i, max(0, i - bandwidth):min(s, i + bandwidth + 1)] = 1
    if is_cauasl:
        _causal_trim_last_batch(m, batch)
    return m


def generate_bigbird_mask(attr_mask, globalwidth=1, bandwidth=1, fill_rate=0.2, is_cauasl=False):
    """src/util/masks.py:86-122 - global + band + seeded random points.

    The random part re-seeds the stdlib generator with 0 and then, per batch and
    per 32-row block i < S/32 - 1, draws the column block with ``choice`` and
    ``int(1024 * fill_rate)`` points with two ``randint(0, 32)`` calls each
    (inclusive upper bound, x before y), in exactly this order.
    """
    b, s = attr_mask.shape[0], attr_mask.shape[1]
    m = np.zeros_like(attr_mask)
    batch = 0
    for batch in range(b):
        m[batch, :globalwidth, :] = 1
        m[batch, :, :globalwidth] = 1
    for batch in range(b):
        for i in range(s):
            m[batch, i, max(0, i - bandwidth):min(s, i + bandwidth + 1)] = 1
    num_ones_in_block = int(1024 * fill_rate)
    random.seed(0)
    nblk = int(s / 32)
    for batch in range(b):
        for i in range(nblk - 1):
            start_x = i * 32
            if i == 0:
                start_y = start_x + 32 * random.choice([1, 0])
            elif i == nblk - 2:
                start_y = start_x + 32 * random.choice([-1, 0])
            else:
                start_y = start_x + 32 * random.choice([-1, 0, 1])
            for _ in range(num_ones_in_block):
                rx = random.randint(0, 32)
                ry = random.randint(0, 32)
                m[batch, start_x + rx, start_y + ry] = 1
    if is_cauasl:
        _causal_trim_last_batch(m, batch)
    return m


def get_sparse_storage(mask, block_size_m, block_size_n):
    """src/util/masks.py:125-184 - dense 0/1 mask (batch 0 only) -> block LUT.

    Row-major walk over (query block, key block): a block of all ones is FULL,
    of all zeros is skipped, anything else is PARTIAL and carries the additive
    fp16 block -10000 * (1 - block).  LOAD lists full and partial blocks merged
    in ascending key-block order.  Returns the same 8-tuple as the reference
    with numpy arrays in place of tensors.
    """
    n = mask.shape[-1]
    full_row_ptr, full_col_idx = [0], []
    part_row_ptr, part_col_idx, part_block_mask = [0], [], []
    load_row_ptr, load_col_idx = [0], []
    nnz = np.float32(np.count_nonzero(mask)) / np.float32(n * n) * 100
    fc = pc = lc = 0
    for i in range(0, n, block_size_m):
        for j in range(0, n, block_size_n):
            block = mask[0, i:i + block_size_m, j:j + block_size_n]
            if np.all(block == 1):
                full_col_idx.append(j // block_size_n)
                fc += 1
                load_col_idx.append(j // block_size_n)
                lc += 1
            elif np.all(block == 0):
                continue
            else:
                add = (np.float16(NEG_MASK) * (np.float16(1.0) - block.astype(np.float16))).astype(np.float16)
                part_col_idx.append(j // block_size_n)
                part_block_mask.append(add)
                pc += 1
                load_col_idx.append(j // block_size_n)
                lc += 1
        full_row_ptr.append(fc)
        part_row_ptr.append(pc)
        load_row_ptr.append(lc)
    i32 = lambda x: np.asarray(x, dtype=np.int32)
    if len(part_block_mask) == 0:
        pbm = np.ones((1, block_size_m, block_size_n), dtype=np.float16)
    else:
        pbm = np.stack(part_block_mask, axis=0)
    return (nnz, i32(full_row_ptr), i32(full_col_idx), i32(part_row_ptr), i32(part_col_idx),
            pbm, i32(load_row_ptr), i32(load_col_idx))


def expand_sparse_storage(lut, n, block_size_m, block_size_n):
    """Inverse of get_sparse_storage: rebuild the dense [n, n] 0/1 mask.

    full -> ones, partial -> (additive block == 0), absent -> zeros.  Used for
    the round-trip invariant; has no counterpart in the reference.
    """
    _, frp, fci, prp, pci, pbm, lrp, lci = lut
    out = np.zeros((n, n), dtype=np.float32)
    for r in range(n // block_size_m):
        for t in range(frp[r], frp[r + 1]):
            c = fci[t]
            out[r * block_size_m:(r + 1) * block_size_m, c * block_size_n:(c + 1) * block_size_n] = 1
        for t in range(prp[r], prp[r + 1]):
            c = pci[t]
            out[r * block_size_m:(r + 1) * block_size_m, c * block_size_n:(c + 1) * block_size_n] = \
                (pbm[t].astype(np.float32) == 0).astype(np.float32)
    return out
