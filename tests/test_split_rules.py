"""How the attention kernels' keys are split between waves and blocks: the rules are plain functions of a step's sizes,
so what every kernel launch assumes of them is checked here for many sizes (the kernels refuse what breaks these,
`csrc/attention_mfma.hip` attention_launch: splits a power of two for the decode kernel, a share that is a multiple of
32 keys, of 64 for the tiled kernel, and splits x share covering the longest context)."""
import itertools

import pytest

from inferrs_amd import ops


@pytest.mark.parametrize("g", [1, 2, 4, 5, 8, 16, 20])
def test_decode_split_covers_the_context_within_one_round_of_the_chip(g):
    for n_seqs, nkv, kv in itertools.product((1, 2, 3, 8, 16, 33, 64, 200), (1, 2, 8), (1, 31, 64, 500, 512, 513, 1024,
                                                                                     2048, 4096, 8192, 40960, 131072)):
        splits, chunk = ops.decode_split(n_seqs, nkv, g, kv)
        assert splits >= 1 and splits & (splits - 1) == 0 and splits <= 128
        assert chunk % 32 == 0 and splits * chunk >= kv
        if splits > 1:
            assert (splits - 1) * 32 < kv, "no more splits than steps of 32 keys (a split may be empty: shorter requests of a batch have such)"
            assert chunk >= 64, "a wave's share is worth two steps of 32 keys"
            items = n_seqs * nkv * -(-g // 16)
            assert items * splits <= ops.DECODE_WAVES, "one round of the chip"
        if kv <= 512:
            assert splits == 1 or chunk >= 128
        if splits > ops.DECODE_MANY_SPLITS:
            assert chunk > 64, "many blocks to merge only for long shares"


def test_decode_split_at_the_measured_points():
    # (32 query and 8 key/value heads; the choices that the measurements in the rule's description name)
    assert ops.decode_split(1, 8, 4, 8192)[0] == 64
    assert ops.decode_split(8, 8, 4, 8192)[0] == 16
    assert ops.decode_split(64, 8, 4, 8192)[0] == 2
    assert ops.decode_split(1, 8, 4, 2048)[0] == 32
    assert ops.decode_split(1, 8, 4, 1024)[0] == 16
    assert ops.decode_split(1, 8, 4, 512)[0] == 4
    assert ops.decode_split(2, 8, 4, 4096)[0] == 32


@pytest.mark.parametrize("d", [64, 128])
def test_prompt_split_covers_the_context(d):
    for n_seqs, nkv, g, q, kv in itertools.product((1, 3, 16), (1, 8), (1, 4, 5), (1, 2, 17, 128, 512, 2048),
                                                   (17, 512, 2048, 8192, 40000)):
        if q > kv:
            continue
        splits, chunk = ops.attention_split(n_seqs, nkv, g, q, kv, d)
        assert 1 <= splits <= 128 and splits * chunk >= kv and chunk % 32 == 0
        tiled = d == 128 and q * g >= ops.ATTN_TILE_COLS
        if tiled:
            assert chunk % 64 == 0, "the tiled kernel walks stages of 64 keys"
            if 2 * q > kv:
                assert splits == 1, "portions that span most of their context keep their keys together"
