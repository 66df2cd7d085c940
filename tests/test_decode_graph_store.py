"""Host logic of the decoder's graph store (no GPU): a slot of the step holds the graph of one owner (a cache or one
of its layers), compared by identity; a new cache replaces the previous one's entries, so the store stays bounded
however many fresh caches pass through."""
import gc
import weakref


def make_decoder():
    from mxfp4_int8_m5_amd import fused_qwen3 as Q
    dec = Q.DecodeQwen3.__new__(Q.DecodeQwen3)
    dec.graphs = {}
    return dec


class Layer:
    pass


class Cache(list):
    pass


def fake_step(dec, cache):
    """What step() does to the store, with strings for graphs: one entry per slot, bound to its owner."""
    slots = [(("step",), cache)] + [(("pre", i), c) for i, c in enumerate(cache)] + [(("post", i), None)
                                                                                      for i in range(len(cache))]
    captured = 0
    for key, owner in slots:
        if dec._lookup(key, owner) is None:
            dec.graphs[key] = ("graph", [], "out", owner)
            captured += 1
    return captured


def test_entry_is_bound_to_the_owner_object():
    dec = make_decoder()
    a = Cache([Layer(), Layer()])
    dec.graphs[("step",)] = ("graph", [], "out", a)
    assert dec._lookup(("step",), a)[0] == "graph"
    b = Cache([Layer()])
    assert dec._lookup(("step",), b) is None          # another object: the entry is dropped, to be captured again
    assert ("step",) not in dec.graphs


def test_fresh_cache_per_prompt_leaves_a_bounded_store_and_frees_the_old_caches():
    dec = make_decoder()
    layers = 3
    refs = []
    for prompt in range(40):
        c = Cache([Layer() for _ in range(layers)])
        refs.append(weakref.ref(c))
        assert fake_step(dec, c) == (1 + 2 * layers if prompt == 0 else 1 + layers)   # owner-less slots are kept
        assert fake_step(dec, c) == 0                                                 # second token: all replays
        assert len(dec.graphs) == 1 + 2 * layers
        del c
    gc.collect()
    assert sum(r() is not None for r in refs) == 1          # only the most recent cache is kept alive


def test_release_drops_the_graphs_of_one_cache():
    dec = make_decoder()
    a = Cache([Layer(), Layer()])
    fake_step(dec, a)
    dec.release(Cache([Layer()]))                            # not the stored cache: nothing happens
    assert len(dec.graphs) == 5
    dec.release(a)
    assert set(dec.graphs) == {("post", 0), ("post", 1)}
    dec.release()
    assert not dec.graphs
