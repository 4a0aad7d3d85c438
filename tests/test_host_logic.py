"""Host-side logic that needs no GPU: knobs and wave-count selection."""
import pytest

from mintccl_amd import common, protocol


def test_reference_constants():
    assert common.NULL == 0 and common.VECTORIZED_BYTES == 16 and common.WARP_SIZE == 64
    assert protocol.BYTES_LL128_MSG == 128 and protocol.BYTES_LL128_RAW == 120
    assert protocol.WORKGROUP_SIZE == 8 and protocol.PAYLOAD_FLAG_THREAD == 8
    assert protocol.BYTES_BLOCK_MSG == 1024 and protocol.BYTES_BLOCK_RAW == 960


def test_env_knobs_are_read_at_call_time(monkeypatch):
    assert common.num_blocks() == 16 and common.num_warps() == 16
    assert common.buff_size() == 4194304 and common.test_count() == 67108864
    monkeypatch.setenv("MINTCCL_NUM_BLOCKS", "32")
    monkeypatch.setenv("MINTCCL_BUFFSIZE", "8388608")
    monkeypatch.setenv("MINTCCL_TEST_MODE", "0")      # any non-empty string (common.py:113)
    assert common.num_blocks() == 32 and common.buff_size() == 8388608
    assert common.test_mode() is True
    monkeypatch.setenv("MINTCCL_PROTOCOL", "simple")
    assert common.protocol_env() == 1


@pytest.mark.parametrize("n,cap,want", [(64, 16, 16), (64, 100, 64), (60, 16, 15), (7, 4, 1),
                                        (512, 128, 128), (1, 5, 1)])
def test_largest_divisor(n, cap, want):
    assert common._largest_divisor_at_most(n, cap) == want
