"""Host model of which carry / prefix slots each kernel variant writes and which it reads.

The forward records, per (row, 32-key sub-tile), the product of (1 - sigma) above the sub-tile (`carry`), the dQ
kernel records the prefix sum of g below it (`prefix`), and the dK/dV kernels start their scans from both.  The
buffers come from the allocator uninitialised, so every slot a dK/dV or dQ variant reads with its math enabled must
have been written by whichever forward / dQ variant ran before it -- for every sequence length, for both
`attend_current` settings and for every pairing of variants the launcher can produce (the forward and the backward
choose between the aligned and the generic kernels independently).  The index arithmetic below restates, variant by
variant, the loop bounds and skip tests of csrc/sba_fwd.hip, sba_bwd_dq.hip and sba_bwd_dkv.hip; the GPU suite
checks the same property on the device by poisoning the buffers with NaN.
"""
import pytest

BQ = 128


def cdiv(a, b):
    return -(-a // b)


def carry_offset(u, m):
    q, r = u >> 2, u & 3
    return u * (m * 128) - 128 * (2 * q * (q - 1) + r * q)


def slot(u, row, m):
    """Flat slot of (sub-tile u, row) in a sequence of m query tiles, with the range checks the layout implies."""
    assert 0 <= u < 4 * m and BQ * (u >> 2) <= row < BQ * m, (u, row, m)
    s = carry_offset(u, m) + (row - BQ * (u >> 2))
    assert 0 <= s < 256 * m * (m + 1)
    return s


def tile_key_steps(L, ac, qt, kt):
    last_row = min(BQ * qt + BQ, L) - 1
    last_key = last_row - 1 + ac
    return 0 if last_key < 0 else last_key // kt + 1


def forward_writes(L, ac, kt):
    m, out = cdiv(L, BQ), set()
    for qt in range(m):
        n = tile_key_steps(L, ac, qt, kt)
        subs = list(range(n)) if kt == 32 else list(range(2 * n))
        if kt == 32 and n % 2 == 1:
            subs.append(n)                      # the product above the upper half of the last 64-key tile
        for u in subs:
            for row in range(BQ * qt, BQ * qt + BQ):
                out.add(slot(u, row, m))
    return out


def dq_prefix_writes(L, ac, kt):
    m, out = cdiv(L, BQ), set()
    for qt in range(m):
        n = tile_key_steps(L, ac, qt, kt)
        for u in (range(n) if kt == 32 else range(2 * n)):
            for row in range(BQ * qt, BQ * qt + BQ):
                out.add(slot(u, row, m))
    return out


def dq_carry_reads(L, ac, kt):
    m, out = cdiv(L, BQ), set()
    for qt in range(m):
        for jt in range(tile_key_steps(L, ac, qt, kt)):
            u = jt if kt == 32 else 2 * jt + 1
            for row in range(BQ * qt, BQ * qt + BQ):
                out.add(slot(u, row, m))
    return out


def dkv_reads(L, ac, variant, rows_beyond_end_count=False):
    """(carry slots, prefix slots) read with the element-wise math enabled."""
    m = cdiv(L, BQ)
    carry, prefix = set(), set()
    last = (lambda w_last: w_last) if rows_beyond_end_count else (lambda w_last: min(w_last, L - 1))
    if variant == "pipelined128":          # 128-key tiles, steps of 32 rows, producer g = sub-tile g
        for j0 in range(0, L, 128):
            first_row = j0 + 1 - ac
            if first_row >= L:
                continue
            row_begin = (first_row // 32) * 32
            for t in range(cdiv(L - row_begin, 32)):
                q0 = row_begin + 32 * t
                for g in range(4):
                    jb = j0 + 32 * g
                    if jb > last(q0 + 31) - 1 + ac or jb >= L:
                        continue
                    for row in range(q0, q0 + 32):
                        carry.add(slot(j0 // 32 + g, row, m))
                        prefix.add(slot(j0 // 32 + g, row, m))
    elif variant == "producer64":          # 64-key tiles, steps of 64 rows, producer (rg, group)
        for j0 in range(0, L, 64):
            first_row = j0 + 1 - ac
            if first_row >= L:
                continue
            row_begin = (first_row // 64) * 64
            for t in range(cdiv(L - row_begin, 64)):
                for rg in range(2):
                    w_first = row_begin + 64 * t + 32 * rg
                    for group in range(2):
                        jb = j0 + 32 * group
                        if jb > last(w_first + 31) - 1 + ac or jb >= L:
                            continue
                        for row in range(w_first, w_first + 32):
                            carry.add(slot(j0 // 32 + group, row, m))
                            prefix.add(slot(j0 // 32 + group, row, m))
    else:                                   # generic: 64-key tiles, 128-row query tiles, a wave per 32 rows
        for j0 in range(0, L, 64):
            first_row = j0 + 1 - ac
            if first_row >= L:
                continue
            for qt in range(first_row // BQ, m):
                for w in range(4):
                    w_first = BQ * qt + 32 * w
                    if j0 > last(w_first + 31) - 1 + ac:
                        continue
                    for row in range(w_first, w_first + 32):
                        carry.add(slot(j0 // 32 + 1, row, m))
                        prefix.add(slot(j0 // 32, row, m))
    return carry, prefix


# (forward key step, dQ key step, dK/dV variant): what the launchers can pair up.
PAIRINGS = [
    (32, 32, "pipelined128"),   # head_dim 128, everything aligned
    (64, 32, "producer64"),     # head_dim 64, everything aligned
    (64, 64, "generic"),        # unaligned / other head_dim
    (32, 64, "generic"),        # head_dim 128: aligned forward, a gradient tensor that forces the generic backward
    (64, 32, "pipelined128"),   # head_dim 128: generic forward (e.g. unaligned o), aligned backward
]


@pytest.mark.parametrize("fwd_kt,dq_kt,dkv", PAIRINGS)
@pytest.mark.parametrize("ac", [0, 1])
def test_every_slot_read_was_written(fwd_kt, dq_kt, dkv, ac):
    lengths = list(range(1, 420)) + [511, 512, 513, 640, 641, 673, 705, 1000]
    for L in lengths:
        written_carry = forward_writes(L, ac, fwd_kt)
        written_prefix = dq_prefix_writes(L, ac, dq_kt)
        assert dq_carry_reads(L, ac, dq_kt) <= written_carry, f"dQ reads an unwritten product, L={L}"
        carry, prefix = dkv_reads(L, ac, dkv)
        assert carry <= written_carry, f"dK/dV reads an unwritten product, L={L}: {sorted(carry - written_carry)[:4]}"
        assert prefix <= written_prefix, f"dK/dV reads an unwritten prefix sum, L={L}: {sorted(prefix - written_prefix)[:4]}"


@pytest.mark.parametrize("L,dq_kt,dkv", [(33, 32, "pipelined128"), (161, 32, "pipelined128"), (97, 32, "producer64")])
def test_model_flags_a_skip_test_that_counts_rows_beyond_the_end(L, dq_kt, dkv):
    """A skip test that lets rows beyond the sequence's end count as seeing a sub-tile (`jb > w_last - 1`) reads
    prefix sums the dQ kernel never wrote when L - 1 is a multiple of 32 but not of 128: the model must tell the two
    skip tests apart, or it pins nothing."""
    written_prefix = dq_prefix_writes(L, 0, dq_kt)
    assert not dkv_reads(L, 0, dkv, rows_beyond_end_count=True)[1] <= written_prefix
    assert dkv_reads(L, 0, dkv)[1] <= written_prefix
