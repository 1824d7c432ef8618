"""How the few-tile GEMM kernels (fp32 GemmF32SkinnyKernel, fp16 GemmF16Few) hand the K range to
a tile's wavefronts: groups of `group_k` values of k, a contiguous run of groups per wavefront,
whole groups in a loop that loads `depth` groups ahead (indices clamped to the wavefront's last
whole group), the group that K ends in read element by element by the one wavefront that owns
it.  The partition arithmetic is the kernels' own (sapphire_amd/csrc/sph_k_partition.h, reached
through the host harness; no device is needed); the loop below is the kernels' loop over it.
Checked: every k is multiplied exactly once, and no load of a whole group reaches past K.
"""
import itertools

import pytest

from tests import host_layer as hl


def wave_plan(K, group_k, waves, depth=4):
    """(multiplied, loaded) per wavefront: lists of (group, whole) and of whole-group indices."""
    plan = []
    for w in range(waves):
        p = hl.k_partition(K, group_k, waves, w, depth)
        multiplied, loaded = [], []
        if p["g_begin"] < p["whole_end"]:
            slots = [hl.k_partition_slot(K, group_k, waves, w, depth, None, d) for d in range(depth)]
            loaded += slots
            g = p["g_begin"]
            while g < p["rounds_end"]:
                for d in range(depth):
                    multiplied.append((slots[d], True))
                    slots[d] = hl.k_partition_slot(K, group_k, waves, w, depth, g, d)
                    loaded.append(slots[d])
                g += depth
            for d in range(depth - 1):
                if p["rounds_end"] + d < p["whole_end"]:
                    multiplied.append((slots[d], True))
        if p["owns_partial"]:
            multiplied.append((p["whole"], False))
        plan.append((multiplied, loaded))
    return plan


@pytest.mark.parametrize("group_k,waves", [(8, 4), (16, 4), (16, 16), (32, 4), (32, 16)])
def test_every_k_is_multiplied_once_and_no_whole_group_passes_k(group_k, waves):
    ks = itertools.chain(range(1, 200), (255, 256, 257, 511, 512, 513, 784, 1000, 1023, 1024,
                                         1025, 4095, 4096, 4097, 8203))
    for K in ks:
        seen = [0] * K
        for multiplied, loaded in wave_plan(K, group_k, waves):
            for g in loaded:
                assert (g + 1) * group_k <= K, (K, g)           # a whole group lies below K
            for g, whole in multiplied:
                if whole:
                    assert (g + 1) * group_k <= K, (K, g)
                for k in range(g * group_k, min((g + 1) * group_k, K)):
                    seen[k] += 1
        assert seen == [1] * K, (K, group_k, waves)


def test_groups_are_multiplied_in_ascending_order_within_a_wavefront():
    """The partial sums meet in wavefront order, and inside a wavefront the groups come in
    ascending k: together that fixes the order of the sum, whatever the timing."""
    for K, group_k, waves in [(1000, 8, 4), (4097, 16, 16), (784, 32, 4), (65, 16, 4)]:
        previous = -1
        for multiplied, _ in wave_plan(K, group_k, waves):
            order = [g for g, _ in multiplied]
            assert order == sorted(order)
            if order:
                assert order[0] > previous
                previous = order[-1]
