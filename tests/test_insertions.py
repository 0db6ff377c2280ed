"""The insertions queue (host logic of lily_insertions_*): the thinking control's answers
(src/thinking.rs:485-608, Action::{Keep, Before, After, Replace}) as per-row forced tokens."""
import pytest

import lily_sampler as LS


def test_after_before_replace_order_and_rows():
    q = LS.Insertions(3)
    assert q.next() == ([None, None, None], 0)
    q.push(0, LS.INSERT_AFTER, drawn=7, ids=[10, 11])
    q.push(2, LS.INSERT_BEFORE, drawn=9, ids=[20])        # 20, then the drawn 9 again
    assert q.pending(0) == 2 and q.pending(1) == 0 and q.pending(2) == 2
    assert q.next() == ([10, None, 20], 2)
    q.push(1, LS.INSERT_REPLACE, drawn=5, ids=[30, 31, 32])
    assert q.next() == ([11, 30, 9], 3)
    assert q.next() == ([None, 31, None], 1)
    q.push(1, LS.INSERT_AFTER, drawn=31, ids=[40])         # lands behind what is still queued
    assert q.next() == ([None, 32, None], 1)
    assert q.next() == ([None, 40, None], 1)
    assert q.next() == ([None, None, None], 0)
    q.close()


def test_clear_and_empty_insertions():
    q = LS.Insertions(2)
    q.push(0, LS.INSERT_AFTER, drawn=1, ids=[2, 3, 4])
    q.clear(0)
    assert q.pending(0) == 0
    q.push(1, LS.INSERT_BEFORE, drawn=8, ids=[])           # nothing but the drawn token again
    assert q.next() == ([None, 8], 1)
    q.push(1, LS.INSERT_REPLACE, drawn=8, ids=[])          # a stop token dropped, nothing in its place
    assert q.next() == ([None, None], 0)
    q.close()


def test_rejections():
    q = LS.Insertions(1)
    with pytest.raises(LS.SamplerError):
        q.push(1, LS.INSERT_AFTER, drawn=0, ids=[1])       # row out of range
    with pytest.raises(LS.SamplerError):
        q.push(0, 7, drawn=0, ids=[1])                     # unknown kind
    with pytest.raises(LS.SamplerError):
        q.push(0, LS.INSERT_AFTER, drawn=0, ids=[LS.NO_TOKEN])
    assert q.pending(5) == 0
    q.close()
