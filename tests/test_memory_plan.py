"""The static activation-memory plan of the benchmark workloads (megengine_amd.workloads.first_fit_offsets): tensors
whose lifetimes overlap never share bytes, and the arena is no larger than the sum and no smaller than the largest live
set.  The liveness rule follows the reference's static allocator (src/core/impl/graph/var_node_mem_mgr/
static_mem_alloc.h:18-40: an interval from the step that writes a variable to the last step that reads it)."""
import numpy as np

from megengine_amd import workloads


def _check(tensors, granule):
    offsets, top = workloads.first_fit_offsets(tensors, granule)
    sizes = [(s + granule - 1) // granule * granule for s, _, _ in tensors]
    assert all(o % granule == 0 for o in offsets)
    assert top == max(o + s for o, s in zip(offsets, sizes))
    n = len(tensors)
    for a in range(n):
        for b in range(a + 1, n):
            (_, wa, ra), (_, wb, rb) = tensors[a], tensors[b]
            ra, rb = max(ra, wa), max(rb, wb)
            if wa <= rb and wb <= ra:  # lifetimes [write, last read] intersect
                assert offsets[a] + sizes[a] <= offsets[b] or offsets[b] + sizes[b] <= offsets[a], (a, b)
    steps = max(max(w, r) for _, w, r in tensors) + 1
    peak = max(sum(sz for sz, (_, w, r) in zip(sizes, tensors) if w <= t <= max(r, w)) for t in range(steps))
    assert peak <= top <= sum(sizes)
    return top, peak


def test_random_lifetimes():
    rng = np.random.RandomState(3)
    for case in range(200):
        n = int(rng.randint(1, 40))
        tensors = []
        for i in range(n):
            tensors.append((int(rng.randint(1, 100000)), i, int(rng.randint(i - 1, min(n, i + 6)))))
        _check(tensors, int(rng.choice([1, 256, 4096])))


def test_chain_reuses_two_buffers():
    # a plain chain: every output is read by the next step only -> two buffers alternate
    tensors = [(1000, i, i + 1) for i in range(10)]
    offsets, top = workloads.first_fit_offsets(tensors, 1)
    assert top == 2000 and sorted(set(offsets)) == [0, 1000]


def test_resnet50_lifetimes():
    """Lifetimes of the ResNet-50 stack from the layer list alone (no tensors): the arena holds a block's input, its
    two inner outputs, its shortcut and its output at most -- well under a third of one buffer per layer."""
    layers = workloads.resnet50(64)
    index = {l.name: i for i, l in enumerate(layers)}
    last = {}
    prev = None
    for i, l in enumerate(layers):
        for name in (l.src if l.src is not None else prev, l.z):
            if name in index:
                last[name] = i
        prev = l.name
    tensors = [(l.n * l.oc * l.oh * l.ow, i, last.get(l.name, i)) for i, l in enumerate(layers)]
    top, peak = _check(tensors, 4096)
    assert top < 0.3 * sum(t[0] for t in tensors)
    assert top <= 1.25 * peak   # first fit is not optimal: 128 MB for a peak of 116 MB
