"""Case lists shared by make_golden.py (which records the reference's answers) and the tests
(which replay them against the oracle and the host layer)."""

# (y shape, a shape, b shape) for Compute::Gemm's walk
PLAN_CASES = [
    ([256, 256], [256, 256], [256, 256]),                    # config 1
    ([16, 512, 512], [16, 512, 512], [1, 512, 512]),          # config 2: B broadcast
    ([4096, 4096], [4096, 4096], [4096, 4096]),               # config 3 shape class
    ([1024, 1024], [1024, 1], [1, 1024]),                     # Linear bias step (K = 1)
    ([1024, 10], [1024, 1024], [1024, 10]),
    ([7, 5, 3], [7, 5, 4], [7, 4, 3]),                        # Gemm1 recipe, all batch dims equal
    ([2, 3, 3, 2], [2, 1, 3, 2], [2, 3, 2, 2]),               # BroadcastWithOneDimension
    ([3, 3, 2], [3, 4], [3, 4, 2]),                           # BroadcastWithMissingDimension
    ([2, 3, 3, 2], [3, 4], [2, 3, 4, 2]),                     # BroadcastMixed
    ([5, 6, 8], [1, 6, 9], [5, 9, 8]),                        # conv-style A broadcast {1,C,K}
    ([4, 2, 2], [2, 3], [4, 3, 2]),
    ([3], [4], [4, 3]),                                       # 1-D operands lifted to [1,n]
    ([2, 2, 3, 4, 5], [2, 1, 3, 4, 6], [1, 2, 3, 6, 5]),
    ([2, 2, 3, 4, 5], [1, 1, 1, 4, 6], [2, 2, 3, 6, 5]),
    ([6, 4, 5], [3, 4, 2], [2, 2, 5]),                        # mismatched leading dims (modulo rule)
    ([2, 4, 5], [6, 4, 2], [3, 2, 5]),                        # output smaller than inputs: repeats
    ([1, 1, 4, 4], [1, 4, 4], [4, 4]),
]

# Compute::Gemm host branch on seeded data: (name, y shape, a shape, b shape, seed)
KAT_OP_CASES = [
    ("plain", [9, 7], [9, 5], [5, 7], 10),
    ("batched", [4, 6, 5], [4, 6, 3], [4, 3, 5], 20),
    ("b_broadcast", [4, 6, 5], [4, 6, 3], [1, 3, 5], 30),
    ("one_dim", [2, 3, 3, 2], [2, 1, 3, 2], [2, 3, 2, 2], 40),
    ("missing_dim", [3, 3, 2], [3, 4], [3, 4, 2], 50),
    ("mixed", [2, 3, 3, 2], [3, 4], [2, 3, 4, 2], 60),
    ("repeats", [2, 4, 5], [6, 4, 2], [3, 2, 5], 70),
    ("vector", [3], [4], [4, 3], 80),
]

# Dense::Naive::Gemm leaf: (name, batch, M, N, K, seed)
KAT_GEMM_CASES = [
    ("tiny", 1, 2, 3, 4, 100),
    ("k1", 2, 8, 5, 1, 110),
    ("odd", 3, 17, 13, 29, 120),
    ("square", 1, 64, 64, 64, 130),
    ("longk", 1, 4, 4, 777, 140),
]

SHAPE_CASES = [[5], [3, 4], [2, 3, 4], [2, 3, 4, 5], [1, 1, 6], [7, 1], [2, 2, 2, 2, 2]]

# Compute::Sub host branch: (name, y shape, a shape, b shape, seed)
SUB_CASES = [
    ("equal", [6, 5], [6, 5], [6, 5], 200),
    ("vector", [37], [37], [37], 210),
    ("b_repeats", [4, 3, 5], [4, 3, 5], [1, 3, 5], 220),
    ("a_repeats", [2, 3, 4, 5], [1, 1, 4, 5], [2, 3, 4, 5], 230),
    ("missing_dim", [3, 4, 5], [3, 4, 5], [4, 5], 240),
    ("last_differs", [3, 4], [3, 4], [3, 1], 250),
]

# Dense::Naive::Sub leaf: (name, totalSize, inputStride, broadcastA, broadcastB, seed)
SUB_LEAF_CASES = [
    ("plain", 101, 0, False, False, 300),
    ("wrap_a", 60, 12, True, False, 310),
    ("wrap_b", 60, 5, False, True, 320),
    ("wrap_both", 64, 16, True, True, 330),
]
