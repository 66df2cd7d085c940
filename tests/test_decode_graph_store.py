"""Host logic of the decoder's graph store (no GPU): a captured graph is bound to the cache object it was captured
for, not to that object's id."""
import gc


def make_decoder():
    from mxfp4_int8_m5_amd import fused_qwen3 as Q
    dec = Q.DecodeQwen3.__new__(Q.DecodeQwen3)
    dec.graphs = {}
    return dec


class Cache(list):
    pass


def test_entry_is_bound_to_the_owner_object_not_to_its_id():
    dec = make_decoder()
    a = Cache([object(), object()])
    key = ("step", id(a))
    dec.graphs[key] = ("graph", [], "out", a)
    assert dec._lookup(key, a)[0] == "graph"
    b = Cache([object()])
    assert dec._lookup(key, b) is None          # same key (a recycled id), another object: the entry is dropped
    assert key not in dec.graphs


def test_store_keeps_the_owner_alive_so_its_id_cannot_be_recycled():
    dec = make_decoder()
    ids = set()
    for _ in range(50):
        c = Cache([object()])
        assert id(c) not in ids
        ids.add(id(c))
        dec.graphs[("step", id(c))] = ("graph", [], "out", c)
        del c
        gc.collect()
    assert len(dec.graphs) == 50


def test_release_drops_the_graphs_of_one_cache():
    dec = make_decoder()
    a, b = Cache([object(), object()]), Cache([object()])
    dec.graphs[("step", id(a))] = ("g", [], "o", a)
    dec.graphs[("pre", 0, id(a[0]))] = ("g", [], "o", a[0])
    dec.graphs[("pre", 1, id(a[1]))] = ("g", [], "o", a[1])
    dec.graphs[("step", id(b))] = ("g", [], "o", b)
    dec.graphs[("post", 0)] = ("g", [], "o", None)
    dec.release(a)
    assert set(dec.graphs) == {("step", id(b)), ("post", 0)}
    dec.release()
    assert not dec.graphs
