"""The position / chunk schedule: the library's host function against the oracle's
restatement of the reference loop, and both against what the schedule must satisfy."""
import itertools

import pytest

import oracle_lib as orc

import ellm_amd


def _reference_last_chunk(prompt_end, chunk):
    """The three lines of src/serving/start copy.rs:71-86 for prompt_begin = 0."""
    remainder = prompt_end % chunk
    last_position, last_interval = prompt_end, chunk
    if remainder == 0:
        last_position -= chunk
    else:
        last_position -= remainder
        last_interval = remainder
    return last_position, last_interval


CASES = list(itertools.product([0, 3, 64], [0, 1, 63, 64, 65, 128, 1000], [1, 7, 64, 4096], [0, 5]))


@pytest.mark.parametrize("begin,length,chunk,generate", CASES)
def test_library_schedule_equals_the_oracle(begin, length, chunk, generate):
    end = begin + length
    want = orc.schedule_calls(begin, end, chunk, end + generate)
    got = ellm_amd.schedule_calls(begin, end, chunk, end + generate)
    assert got == want


@pytest.mark.parametrize("begin,length,chunk,generate", CASES)
def test_schedule_properties(begin, length, chunk, generate):
    end = begin + length
    calls = orc.schedule_calls(begin, end, chunk, end + generate)
    prompt = [c for c in calls if c[0] < end]
    decode = [c for c in calls if c[0] >= end]
    # the prompt calls tile [begin, end) exactly once, in order, each at most one chunk long,
    # and only the last may be shorter
    pos = begin
    for i, (p, n) in enumerate(prompt):
        assert p == pos and 1 <= n <= chunk
        if i + 1 < len(prompt):
            assert n == chunk
        pos += n
    assert pos == end
    assert len(prompt) == (length + chunk - 1) // chunk
    # then one position at a time
    assert decode == [(end + i, 1) for i in range(generate)]


@pytest.mark.parametrize("prompt_end,chunk", [(1, 64), (64, 64), (65, 64), (4096, 512), (4097, 512), (99, 7)])
def test_last_chunk_is_the_reference_one(prompt_end, chunk):
    calls = orc.schedule_calls(0, prompt_end, chunk, prompt_end)
    assert calls[-1] == _reference_last_chunk(prompt_end, chunk)


def test_capacity_and_bad_arguments():
    assert orc.schedule_calls(0, 100, 10, 105, capacity=14) is None          # 10 + 5 calls
    assert len(orc.schedule_calls(0, 100, 10, 105, capacity=15)) == 15
    with pytest.raises(ellm_amd.EllmError):
        ellm_amd.schedule_calls(0, 10, 0, 10)                                  # chunk 0
    with pytest.raises(ellm_amd.EllmError):
        ellm_amd.schedule_calls(10, 5, 4, 20)                                  # end before begin
