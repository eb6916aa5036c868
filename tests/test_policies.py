"""Decisions the host takes about a launch, checked without a GPU: how many workgroups share the keys
of a decode step's requests."""
import pytest

from tiny_llm_amd.kernels import ops


@pytest.fixture
def waves(monkeypatch):
    # eight waves a workgroup up to heads of 64, four beyond (what the library answers on the GPU)
    monkeypatch.setattr(ops, "flash_waves", lambda head_dim, groups=1 << 20: 8 if head_dim <= 64 else 4)


def test_short_contexts_are_not_split(waves):
    for rows in (1, 8, 64):
        assert ops.decode_key_splits(rows, 1024, 4, 64) == 1          # 16 key tiles: two a wave
        assert ops.decode_key_splits(rows, 512, 8, 128) == 1          # 8 key tiles: two a wave


def test_one_request_is_split_down_to_a_tile_a_wave_within_64(waves):
    assert ops.decode_key_splits(1, 2048, 4, 64) == 4
    assert ops.decode_key_splits(1, 8192, 4, 64) == 16
    assert ops.decode_key_splits(1, 32768, 4, 64) == 64
    assert ops.decode_key_splits(1, 1 << 20, 4, 64) == 64
    assert ops.decode_key_splits(1, 131072, 8, 128) == 32             # 8 kv heads: 256 workgroups


def test_splits_stay_within_one_round_of_workgroups_where_one_is_enough(waves):
    for rows, kv, hd in ((8, 4, 64), (8, 8, 128), (16, 8, 128), (64, 4, 64)):
        for ctx in (2048, 8192, 131072):
            assert rows * kv * ops.decode_key_splits(rows, ctx, kv, hd) <= 256


def test_a_mostly_empty_last_round_is_split_away_at_long_contexts(waves):
    # 8 requests x 40 kv heads: 320 workgroups are two rounds for the work of 1.25
    assert ops.decode_key_splits(8, 2048, 40, 128) == 1               # too short to pay for a merge
    assert ops.decode_key_splits(8, 8192, 40, 128) == 4
    assert ops.decode_key_splits(8, 131072, 40, 128) == 4
    # 64 x 8 = 512 workgroups are two full rounds: nothing to gain
    assert ops.decode_key_splits(64, 131072, 8, 128) == 1


def test_more_context_never_means_fewer_splits(waves):
    for rows, kv, hd in ((1, 4, 64), (8, 4, 64), (8, 40, 128), (16, 8, 128), (3, 5, 96)):
        got = [ops.decode_key_splits(rows, ctx, kv, hd) for ctx in (64, 640, 1280, 4224, 8192, 32768, 131072)]
        assert got == sorted(got) and 1 <= got[0] and got[-1] <= 64


def test_prompt_portions_split_their_keys_where_it_was_measured_to_pay():
    heads = dict(num_heads=32, num_kv_heads=8)
    assert ops.prefill_key_splits(2048, 2048, tile_waves=8, **heads) == 1          # a whole prompt: enough workgroups
    assert ops.prefill_key_splits(512, 512, tile_waves=4, **heads) == 1            # 8 key tiles: too short
    assert ops.prefill_key_splits(512, 8192, tile_waves=4, **heads) == 4
    assert ops.prefill_key_splits(512, 131072, tile_waves=4, **heads) == 8         # from 32,768 tokens of context on
    assert ops.prefill_key_splits(2048, 32768, tile_waves=8, **heads) == 1
    assert ops.prefill_key_splits(8192, 131072, tile_waves=8, **heads) == 4        # the same quarter of the keys together
    assert ops.prefill_key_splits(131072, 131072, tile_waves=8, **heads) == 1      # a whole prompt of that length
    for rows in (16, 100, 512, 2048, 8192):
        for ctx in (rows, 4096, 32768, 131072):
            if ctx >= rows:
                assert 1 <= ops.prefill_key_splits(rows, ctx, tile_waves=4, **heads) <= 8
