"""The Python `Buffer`'s pool of dispatch outputs: a set of tensors is offered again only when nothing but the
pool refers to any of them or to their storage (names, tuples, views, dtype reinterpretations all count), so a
caller cannot tell a recycled tensor from the fresh ones the reference allocates; otherwise the call gets fresh
tensors.  Plain CPU tensors: the rule does not depend on the device."""
import torch

from mooncake_amd.mooncake_ep_buffer import _OutputPool


def make():
    return [torch.empty(4, 8), torch.empty(3, dtype=torch.int32), torch.empty((2, 3, 4)).transpose(1, 2)]


def ids(tensors):
    return [id(t) for t in tensors]


def test_a_released_set_is_offered_again_and_a_held_one_is_not():
    pool = _OutputPool()
    a = pool.take(("k",), make)
    first = ids(a)
    b = pool.take(("k",), make)                 # a is still held: fresh tensors
    assert ids(b) != first
    del a
    c = pool.take(("k",), make)                 # a's set has been let go
    assert ids(c) == first
    assert pool.take(("other shape",), make) is not None and ids(pool.take(("other shape",), make)) != first


def test_one_name_or_one_view_keeps_a_set_out_of_circulation():
    pool = _OutputPool()
    a = pool.take(("k",), make)
    first = ids(a)
    kept = a[1]                                 # one tensor of the set still has a name
    del a
    b = pool.take(("k",), make)
    assert ids(b) != first
    del kept
    second = ids(b)
    row = b[0][1]                               # a view: no tensor of the set is named, its storage is in use
    del b
    c = pool.take(("k",), make)
    assert ids(c) == first                      # the first set is free again, the second is not
    d = pool.take(("k",), make)
    assert ids(d) not in (first, second)
    reinterpreted = d[2].view(torch.int32)      # the column-major scales read as integers
    third = ids(d)
    del d, row
    e = pool.take(("k",), make)
    assert ids(e) == second
    f = pool.take(("k",), make)
    assert ids(f) != third
    del reinterpreted


def test_the_pool_holds_a_bounded_number_of_sets():
    pool = _OutputPool()
    held = [pool.take(("k",), make) for _ in range(_OutputPool.limit + 3)]
    assert len({tuple(ids(h)) for h in held}) == len(held)      # all different, none recycled while held
    assert len(pool._sets[("k",)]) == _OutputPool.limit
