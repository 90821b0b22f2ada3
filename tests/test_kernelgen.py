"""Plan generation on the host (no GPU): properties every kernel plan must have."""
from jaxjs_hip import DType
from jaxjs_hip.kernelgen import generate


def test_every_contraction_shape_gets_a_plan():
    """Plan generation must not raise whatever the extents: rows and columns from 2 to 14336 across the tile sizes, k
    from 32 to 8192 (multiples of the slab depths and not), both layouts of B, float16 and float32.  (A k split folded
    inside the launch used to be chosen for tiles that only the general template can run, which has no such fold.)"""
    import random
    from jaxjs_hip.lowering import matmulKernel
    rng = random.Random(1)
    shapes = [(100, 14336, 4096), (65, 4096, 4096), (127, 14336, 4096), (96, 1000, 4096), (8192, 100, 4096), (300, 300, 8192)]
    rows = [2, 33, 64, 65, 100, 128, 129, 200, 256, 300, 1000, 4096]
    for _ in range(60):
        shapes.append((rng.choice(rows), rng.choice(rows + [14336]), rng.choice([32, 64, 100, 256, 768, 1000, 2048, 4096, 4100, 8192])))
    for dt in (DType.Float16, DType.Float32):
        for shape in shapes:
            for bt in (False, True):
                ks = generate(matmulKernel(*shape, dt, b_transposed=bt), "fast")
                assert ks.steps and ks.sources, (dt, shape, bt)
