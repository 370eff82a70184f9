"""Host-side bounds that keep kernels inside their tables, checked against the kernels'
own arithmetic redone in Python."""
import numpy as np

from litinfer_amd.kernels import ops


def pages_touched_by_a_split(p, window, nsplit, page_size, split, given=None, max_blocks=None):
    """As paged_attention_decode_mfma_kernel cuts the keys of the query at position p; `given`: the run
    length a batch of unequal contexts brings (never shorter than this token needs, never longer than
    the table's width would need)."""
    lo = p - window + 1 if window > 0 and p - window + 1 > 0 else 0
    nkeys = p - lo + 1
    per = (-(-nkeys // nsplit) + 31) & ~31
    if given is not None:
        widest = max_blocks * page_size
        if 0 < window < widest:
            widest = window
        cap = (-(-widest // nsplit) + 31) & ~31
        per = max(per, min((given + 31) & ~31, cap))
    k_begin = lo + split * per
    k_end = min(k_begin + per, p + 1)
    if k_begin >= k_end:
        return 0
    return (k_end - 1) // page_size - k_begin // page_size + 1


def test_decode_split_bound_covers_every_split_of_every_context():
    rng = np.random.default_rng(0)
    for _ in range(3000):
        page = int(rng.choice([1, 2, 7, 8, 16, 32, 128]))
        max_blocks = int(rng.integers(1, 5000))
        window = int(rng.choice([0, 0, rng.integers(1, 4000)]))
        nsplit = int(rng.integers(1, 65))
        bound = ops.decode_split_blocks(max_blocks, page, window, nsplit)
        for ctx in {max_blocks * page, int(rng.integers(1, max_blocks * page + 1)), max(1, max_blocks * page - 31)}:
            worst = max(pages_touched_by_a_split(ctx - 1, window, nsplit, page, s) for s in range(nsplit))
            assert worst <= bound, (page, max_blocks, window, nsplit, ctx)
            given = int(rng.integers(0, 2 * max_blocks * page + 64))
            worst = max(pages_touched_by_a_split(ctx - 1, window, nsplit, page, s, given, max_blocks) for s in range(nsplit))
            assert worst <= bound, (page, max_blocks, window, nsplit, ctx, given)
    # pages of one token: 64 splits of 1,024 keys fill the kernel's table exactly, one key more does not fit
    assert ops.decode_split_blocks(64 * 1024, 1, 0, 64) == ops.DECODE_TABLE_CAP
    assert ops.decode_split_blocks(64 * 1024 + 1, 1, 0, 64) > ops.DECODE_TABLE_CAP


def test_the_decode_kernels_float_quotient_is_the_page_of_every_key():
    """paged_attention_decode_mfma_kernel finds a key's page as int((key + 0.5f) * (1.0f / page_size)) in
    float32; redone here with numpy's float32 for every key the host lets through, at page sizes of every kind."""
    keys = np.arange(0, (1 << 21) + 1, dtype=np.int64)
    half = np.float32(0.5)
    for page in (1, 2, 3, 5, 7, 12, 16, 17, 48, 64, 100, 127, 128, 255, 1000, 4097, 65535, 65536):
        inv = np.float32(1.0) / np.float32(page)
        blk = ((keys.astype(np.float32) + half) * inv).astype(np.int64)
        assert np.array_equal(blk, keys // page), page
