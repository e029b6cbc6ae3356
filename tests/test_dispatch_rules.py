"""Launch decisions that are made on the host, as far as they are plain arithmetic (no GPU)."""
import inspect

from ferrox_amd import ops


def splits(n_items, n_heads, n_kv_heads, max_kv_len, cus=256):
    chunk = ops.decode_attention_chunk(n_items, n_heads, n_kv_heads, max_kv_len, cus)
    assert chunk % 64 == 0 and chunk >= 64
    return -(-max_kv_len // chunk)


def test_decode_attention_chunks_fill_the_gpu_and_avoid_partial_rounds():
    # few (sequence, kv head) pairs: chunks enough for about eight waves a CU
    assert splits(1, 16, 16, 2560) >= 12
    assert splits(8, 16, 16, 2560) == 2
    assert splits(8, 28, 4, 2560) == 8
    # as many pairs as CUs, or a whole number of rounds of them: one chunk, no merge launch
    for n in (16, 32, 64):
        assert splits(n, 16, 16, 2560) == 1
    assert splits(128, 28, 4, 2560) == 1
    # a last round far from full (steps recorded for 24, 40, 48 and 56 sequences of 16 kv heads): eight chunks
    for n in (24, 40, 48, 56):
        assert splits(n, 16, 16, 2560) == 8
    assert splits(80, 28, 4, 2560) == 8
    # short sequences have too few tiles to cut, and from four pairs a CU on one chunk is level with the rest
    assert splits(24, 16, 16, 512) == 1
    for n in (72, 96, 128, 256):
        assert splits(n, 16, 16, 2560) == 1
    # another GPU: the same decisions by its own number of CUs
    assert splits(8, 16, 16, 2560, cus=128) == 1 and splits(12, 16, 16, 2560, cus=128) == 8


def test_the_chunk_rule_leaves_the_callers_arguments_alone():
    """The rule counts waves per block; it once did so in a variable named like the `waves` argument of
    `attention_decode`, which then reached the launch instead of the caller's value."""
    src = inspect.getsource(ops.attention_decode)
    body = src[src.index('"""', src.index('"""') + 3):]
    assert "waves =" not in body and "waves=" not in body.replace("int(waves)", "")
    assert "int(waves)" in body
