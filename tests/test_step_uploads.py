"""The ring of pinned buffers a step's numbers travel through (`engine.runner._StepUploads`), on the CPU: what is laid down and
not yet sent goes over with the next piece that is sent or with `flush`, pieces a caller copies itself are left alone, and a
step that brings more than the ring holds still gets its arrays."""
import numpy as np
import torch

from geneinfer_amd.engine.runner import _StepUploads


def test_pieces_laid_down_go_over_with_the_next_one_sent():
    up = _StepUploads("cpu", capacity=64)
    up.begin_step()
    a, b = up.put(np.arange(5), np.arange(10, 13), send=False)
    assert up.sent == 0 and up.used > 0                                  # nothing has gone over yet
    c = up.put(np.arange(20, 27))                                        # ... now everything has, in one copy
    assert up.sent == up.used
    assert a.tolist() == [0, 1, 2, 3, 4] and b.tolist() == [10, 11, 12] and c.tolist() == list(range(20, 27))
    assert all(t.dtype == torch.int32 for t in (a, b, c))
    assert {a.data_ptr() % 16, b.data_ptr() % 16, c.data_ptr() % 16} == {0}      # pieces start at multiples of 16 bytes


def test_flush_sends_what_is_left_and_only_that():
    up = _StepUploads("cpu", capacity=64)
    up.begin_step()
    first = up.put(np.array([1, 2, 3]))
    held = up.put(np.array([7, 8]), send=False)
    up.dev[up.turn][:up.used] = -1                                       # (what the device holds so far, spoilt on purpose)
    up.flush()
    assert held.tolist() == [7, 8] and first.tolist() == [-1, -1, -1]    # only the piece not yet sent was copied
    up.flush()                                                           # nothing left: nothing happens
    assert up.sent == up.used


def test_pieces_for_the_callers_own_copies_are_not_the_rings_to_send():
    up = _StepUploads("cpu", capacity=64)
    up.begin_step()
    staged = up.stage(np.array([4, 5, 6]))
    assert staged.tolist() == [4, 5, 6] and up.sent == up.used           # nothing pending before it: it is skipped
    region = up.region(6)
    region[:] = torch.arange(6, dtype=torch.int32)
    assert up.sent == up.used
    pending = up.put(np.array([9]), send=False)
    staged_later = up.stage(np.array([1, 1]))                            # behind a pending piece: a later flush copies it too, harmlessly
    up.flush()
    assert pending.tolist() == [9] and staged_later.tolist() == [1, 1]


def test_a_step_larger_than_the_ring_still_gets_its_arrays():
    up = _StepUploads("cpu", capacity=8)
    up.begin_step()
    small = up.put(np.array([1, 2]), send=False)
    big_a, big_b = up.put(np.arange(100), np.arange(3))                  # does not fit: ordinary copies, the pending piece stays pending
    assert big_a.tolist() == list(range(100)) and big_b.tolist() == [0, 1, 2]
    up.flush()
    assert small.tolist() == [1, 2]
    assert up.stage(np.arange(50)).tolist() == list(range(50)) and up.region(50).numel() == 50


def test_every_step_takes_the_next_buffer_of_the_ring():
    up = _StepUploads("cpu", capacity=16)
    seen = []
    for step in range(2 * up.DEPTH):
        up.begin_step()
        t = up.put(np.array([step]))
        seen.append((up.turn, t.data_ptr()))
        up.end_step()
    assert [turn for turn, _ in seen[:up.DEPTH]] == [(i + 1) % up.DEPTH for i in range(up.DEPTH)]
    assert [p for _, p in seen[:up.DEPTH]] == [p for _, p in seen[up.DEPTH:]] and len({p for _, p in seen}) == up.DEPTH
