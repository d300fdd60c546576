"""The static activation-memory plan of the benchmark workloads (megengine_amd.workloads.first_fit_offsets): tensors
whose lifetimes overlap never share bytes, and the arena is no larger than the sum and no smaller than the largest live
set.  The liveness rule follows the reference's static allocator (src/core/impl/graph/var_node_mem_mgr/
static_mem_alloc.h:18-40: an interval from the step that writes a variable to the last step that reads it)."""
import numpy as np

from megengine_amd import workloads


def _check(tensors, granule):
    offsets, top = workloads.first_fit_offsets(tensors, granule)
    sizes = [(t[0] + granule - 1) // granule * granule for t in tensors]
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


def test_output_takes_over_a_residual_read_for_the_last_time():
    # 0, 1 and 2 are all read by 3, which reads 0 (its residual) for the last time: with take-over 3 lands on 0's range
    tensors = [(1000, 0, 3), (1000, 1, 3), (1000, 2, 3), (1000, 3, 4, 0), (500, 4, 4)]
    offsets, top = workloads.first_fit_offsets(tensors, 1)
    assert offsets[3] == offsets[0] and top == 3000
    plain, top_plain = workloads.first_fit_offsets([t[:3] for t in tensors], 1)
    assert plain[3] != plain[0] and top_plain == 4000
    # no take-over when the residual is read again later, or sizes differ
    later = [(1000, 0, 4), (1000, 1, 3), (1000, 2, 3), (1000, 3, 4, 0), (500, 4, 4)]
    off2, _ = workloads.first_fit_offsets(later, 1)
    assert off2[3] != off2[0]
    other = [(1000, 0, 3), (1000, 1, 3), (1000, 2, 3), (900, 3, 4, 0)]
    off3, _ = workloads.first_fit_offsets(other, 1)
    assert off3[3] != off3[0]
    # everything else keeps the no-overlap rule
    _check([t[:3] for t in tensors], 1)


def test_resnet50_with_residuals_in_place():
    """With each block's output written over the residual it adds, the arena drops to a block's input, its two inner
    outputs and its shortcut."""
    layers = workloads.resnet50(64)
    index = {l.name: i for i, l in enumerate(layers)}
    last, prev = {}, None
    for i, l in enumerate(layers):
        for name in (l.src if l.src is not None else prev, l.z):
            if name in index:
                last[name] = i
        prev = l.name
    specs = []
    for i, l in enumerate(layers):
        over = index[l.z] if l.z in index and last[l.z] == i else None
        specs.append((l.n * l.oc * l.oh * l.ow, i, last.get(l.name, i), over))
    offsets, top = workloads.first_fit_offsets(specs, 4096)
    _, top_plain = workloads.first_fit_offsets([t[:3] for t in specs], 4096)
    assert top < 0.7 * top_plain
    taken = [i for i, t in enumerate(specs) if t[3] is not None and offsets[i] == offsets[t[3]]]
    assert len(taken) == 16   # every block's last layer
    # apart from the taken-over pairs, live tensors never share bytes
    for a in range(len(specs)):
        for b in range(a + 1, len(specs)):
            if b in taken and specs[b][3] == a:
                continue
            (sa, wa, ra), (sb, wb, rb) = specs[a][:3], specs[b][:3]
            ra, rb = max(ra, wa), max(rb, wb)
            if wa <= rb and wb <= ra:
                assert offsets[a] + sa <= offsets[b] or offsets[b] + sb <= offsets[a], (a, b)
