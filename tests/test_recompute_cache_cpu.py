"""Bookkeeping of the recompute cache without a GPU: which kept run a call may take over (keys, order, signature),
the verification of unkeyed take-overs, and the bounds on what is held.  (The kernels are not involved: the cache
handles tensors it is given.)"""
import pytest
import torch


def _cache(**kw):
    from rwkv_wkv_hip import ops
    return ops, ops.RecomputeCache(**kw)


def _payload(n):
    return (torch.full((n,), 1.0), torch.zeros(4), None, 2)


def test_unkeyed_is_last_in_first_out_by_signature():
    ops, c = _cache()
    r = [torch.randn(3000) for _ in range(3)]
    for i, x in enumerate(r):
        c.push(None, ("sig", 1), x, _payload(10 + i))
    assert c.pop(None, ("sig", 2), r[2]) is None                 # another signature: no take-over, nothing dropped
    assert len(c.entries) == 3
    for i in (2, 1, 0):
        assert c.pop(None, ("sig", 1), r[i])[0].numel() == 10 + i
    assert c.pop(None, ("sig", 1), r[0]) is None and c.bytes == 0
    c.check()                                                    # every take-over met its own inputs


def test_unkeyed_take_over_with_other_inputs_raises_on_check():
    ops, c = _cache()
    a, b = torch.randn(5000), torch.randn(5000)
    c.push(None, "s", a, _payload(8))
    assert c.pop(None, "s", b) is not None                       # taken over (the match is by order and signature) ...
    with pytest.raises(ops.WKVError, match="different inputs"):
        c.check()                                                # ... and reported
    c.check()                                                    # the flag is cleared by the check


def test_keyed_matches_only_its_key():
    ops, c = _cache()
    x = torch.randn(2000)
    c.push(("layer", 0), "s", x, _payload(5))
    c.push(("layer", 1), "s", x, _payload(6))
    c.push(None, "s", x, _payload(7))
    assert c.pop(("layer", 2), "s", x) is None
    assert c.pop(("layer", 0), "t", x) is None
    assert c.pop(("layer", 0), "s", x)[0].numel() == 5            # not the most recent one: found by key
    assert c.pop(None, "s", x)[0].numel() == 7
    assert c.pop(None, "s", x) is None                           # the remaining kept run is keyed: not for an unkeyed call
    assert len(c.entries) == 1


def test_bounds_drop_the_oldest():
    ops, c = _cache(max_entries=2)
    x = torch.randn(100)
    for i in range(4):
        c.push(i, "s", x, _payload(i + 1))
    assert [e[0] for e in c.entries] == [2, 3]
    ops, c = _cache(max_bytes=3 * 4 * 10)
    for i in range(4):
        c.push(i, "s", x, (torch.zeros(10),))                    # 40 bytes each
    assert [e[0] for e in c.entries] == [1, 2, 3] and c.bytes == 120
    c.clear()
    assert c.bytes == 0 and not c.entries


def test_context_managers_nest_and_restore():
    from rwkv_wkv_hip import ops
    assert ops._cache is None and ops._key is None
    with ops.recompute_cache() as outer:
        with ops.call_key("a"):
            assert ops._key == "a"
            with ops.call_key("b"):
                assert ops._key == "b"
            assert ops._key == "a"
        with ops.recompute_cache() as inner:
            assert ops._cache is inner
        assert ops._cache is outer
    assert ops._cache is None and ops._key is None
