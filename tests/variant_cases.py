"""Which shapes reach which compiled variant of the two grouped-product kernels.

The library holds one variant of qmm_small_kernel (streamed segments) per combination of
<bits, SwiGLU fused, waves that split K, unconditional ring, slabs, token groups, ring depth, two row tiles>
and one of qmm_large_kernel (tiled segments) per <bits, SwiGLU fused, tile rows / 64>.  The table below
gives, for every variant, a block (hidden, intermediate, experts, top_k, tokens, bits) whose forward
launches it WITH rows to work on; it was found with the library's launch planner
(mi_moe_debug_plan_forward), which needs no GPU.  tests/test_launch_plan.py checks on any machine that the
table still says what the launch rules do; tests/test_gpu_variants.py runs every case against the oracle
and then asserts that no variant of the library is left without such a launch.
"""

# ((hidden, intermediate, experts, top_k, tokens, bits), variants the case is in the table for)
BLOCK_CASES = [
    ((128, 128, 1, 1, 1, 8), ('qmm_small_kernel<8,0,1,0,0,1,4,0>', 'qmm_small_kernel<8,1,1,0,0,1,4,0>')),
    ((128, 128, 1, 1, 1, 4), ('qmm_small_kernel<4,0,1,0,0,1,4,0>', 'qmm_small_kernel<4,1,1,0,0,1,4,0>')),
    ((128, 128, 1, 1, 9, 4), ('qmm_small_kernel<4,0,1,0,0,2,4,1>', 'qmm_small_kernel<4,1,1,0,0,2,4,0>')),
    ((128, 128, 1, 1, 17, 4), ('qmm_large_kernel<4,0,1>', 'qmm_large_kernel<4,1,1>')),
    ((128, 128, 1, 1, 17, 8), ('qmm_large_kernel<8,0,1>', 'qmm_large_kernel<8,1,1>')),
    ((256, 128, 1, 1, 1, 8), ('qmm_small_kernel<8,1,2,0,0,1,4,0>',)),
    ((128, 256, 1, 1, 1, 8), ('qmm_small_kernel<8,0,2,0,0,1,4,0>',)),
    ((512, 128, 1, 1, 1, 4), ('qmm_small_kernel<4,1,2,0,0,1,4,0>',)),
    ((128, 512, 1, 1, 1, 8), ('qmm_small_kernel<8,0,4,0,0,1,4,0>',)),
    ((128, 512, 1, 1, 1, 4), ('qmm_small_kernel<4,0,2,0,0,1,4,0>',)),
    ((512, 128, 1, 1, 1, 8), ('qmm_small_kernel<8,1,4,0,0,1,4,0>',)),
    ((128, 1024, 1, 1, 1, 4), ('qmm_small_kernel<4,0,4,0,0,1,4,0>',)),
    ((1024, 128, 1, 1, 1, 4), ('qmm_small_kernel<4,1,4,0,0,1,4,0>',)),
    ((3072, 128, 1, 1, 5, 8), ('qmm_small_kernel<8,1,4,1,0,1,8,0>',)),
    ((3072, 128, 1, 1, 5, 4), ('qmm_small_kernel<4,1,4,1,0,1,4,0>',)),
    ((128, 1536, 1, 1, 16, 8), ('qmm_small_kernel<8,0,4,1,0,1,8,0>',)),
    ((128, 2560, 1, 1, 8, 4), ('qmm_small_kernel<4,0,4,1,0,1,4,0>',)),
    ((128, 4096, 1, 1, 6, 8), ('qmm_small_kernel<8,0,4,1,0,1,16,0>',)),
    ((4096, 128, 1, 1, 6, 8), ('qmm_small_kernel<8,1,4,1,0,1,16,0>',)),
    ((5120, 128, 1, 1, 12, 8), ('qmm_small_kernel<8,1,1,1,1,1,8,0>',)),
    ((15360, 128, 1, 1, 1, 8), ('qmm_small_kernel<8,1,4,1,1,1,4,0>',)),
    ((15360, 128, 1, 1, 1, 4), ('qmm_small_kernel<4,1,1,1,0,1,4,0>',)),
    ((7168, 128, 1, 1, 8, 4), ('qmm_small_kernel<4,1,1,1,1,1,4,0>',)),
    ((128, 7168, 1, 1, 8, 4), ('qmm_small_kernel<4,0,1,1,1,1,4,0>',)),
    ((128, 7168, 1, 1, 9, 8), ('qmm_small_kernel<8,0,1,1,1,1,8,0>',)),
    ((128, 6144, 1, 1, 12, 8), ('qmm_small_kernel<8,0,4,1,1,1,8,0>',)),
    ((6144, 128, 1, 1, 12, 8), ('qmm_small_kernel<8,1,4,1,1,1,8,0>',)),
    ((128, 8192, 1, 1, 8, 4), ('qmm_small_kernel<4,0,4,1,1,1,4,0>',)),
    ((128, 13312, 1, 1, 4, 8), ('qmm_small_kernel<8,0,4,1,1,1,4,0>',)),
    ((12288, 128, 1, 1, 5, 4), ('qmm_small_kernel<4,1,4,1,1,1,4,0>',)),
    ((128, 1536, 32, 1, 64, 8), ('qmm_small_kernel<8,0,2,1,0,1,8,0>',)),
    ((1536, 128, 32, 1, 64, 8), ('qmm_small_kernel<8,1,2,1,0,1,8,0>',)),
    ((2048, 1536, 8, 1, 16, 8), ('qmm_small_kernel<8,0,1,1,0,1,8,0>', 'qmm_small_kernel<8,1,2,1,1,1,4,0>')),
    ((256, 2048, 16, 2, 16, 8), ('qmm_small_kernel<8,0,2,1,0,1,16,0>',)),
    ((2048, 256, 16, 4, 12, 8), ('qmm_small_kernel<8,1,2,1,0,1,16,0>',)),
    ((2560, 128, 32, 1, 64, 4), ('qmm_small_kernel<4,1,2,1,0,1,4,0>',)),
    ((256, 2560, 16, 2, 16, 4), ('qmm_small_kernel<4,0,2,1,0,1,4,0>',)),
    ((768, 1536, 16, 2, 16, 8), ('qmm_small_kernel<8,0,2,1,1,1,4,0>',)),
    ((128, 12288, 1, 1, 129, 4), ('qmm_large_kernel<4,1,2>',)),
    ((128, 12288, 1, 1, 129, 8), ('qmm_large_kernel<8,1,2>',)),
    ((128, 2048, 128, 1, 256, 8), ('qmm_small_kernel<8,0,1,1,0,1,16,0>',)),
    ((6144, 128, 32, 1, 160, 8), ('qmm_small_kernel<8,1,2,1,1,1,8,0>',)),
    ((2560, 3072, 4, 1, 12, 4), ('qmm_small_kernel<4,0,2,1,1,1,4,0>',)),
    ((1536, 1536, 16, 1, 32, 8), ('qmm_small_kernel<8,0,1,1,1,1,4,0>',)),
    ((1024, 5120, 4, 2, 16, 8), ('qmm_small_kernel<8,0,2,1,1,1,8,0>',)),
    ((10240, 1024, 4, 1, 8, 4), ('qmm_small_kernel<4,1,2,1,1,1,4,0>',)),
    ((512, 2560, 32, 8, 8, 4), ('qmm_small_kernel<4,0,1,1,0,1,4,0>',)),
    ((1536, 512, 64, 4, 32, 8), ('qmm_small_kernel<8,1,1,1,1,1,4,0>',)),
    ((16384, 2048, 1, 1, 9, 4), ('qmm_small_kernel<4,0,1,1,0,2,4,1>',)),
    ((128, 12288, 1, 1, 300, 4), ('qmm_large_kernel<4,1,4>',)),
    ((128, 12288, 1, 1, 300, 8), ('qmm_large_kernel<8,1,4>',)),
    ((13312, 128, 1, 1, 300, 4), ('qmm_large_kernel<4,0,2>',)),
    ((13312, 128, 1, 1, 300, 8), ('qmm_large_kernel<8,0,2>',)),
    ((2560, 2048, 16, 4, 8, 8), ('qmm_small_kernel<8,1,1,1,0,1,8,0>',)),
    ((16384, 2560, 1, 1, 9, 4), ('qmm_small_kernel<4,0,1,1,0,2,4,0>',)),
    ((16384, 4096, 1, 1, 16, 4), ('qmm_small_kernel<4,0,1,1,1,2,4,0>',)),
    ((16384, 128, 1, 1, 600, 4), ('qmm_large_kernel<4,0,4>',)),
    ((16384, 128, 1, 1, 600, 8), ('qmm_large_kernel<8,0,4>',)),
    ((1536, 512, 64, 8, 48, 4), ('qmm_small_kernel<4,1,1,1,1,2,4,0>',)),
    ((1920, 1024, 32, 1, 256, 4), ('qmm_small_kernel<4,1,1,1,0,2,4,0>',)),
]

# the one variant no block reaches (a plain product whose N is not a multiple of 32, two token groups):
# gather_qmm with N = 48, K = 128, twelve rows for one expert
OP_CASE = dict(N=48, K=128, bits=4, rows=12, variant="qmm_small_kernel<4,0,1,0,0,2,4,0>")


def rules(H, I, E, k, T, bits):
    """(tile lists are built, rows from which a segment is tiled): the library's own rule."""
    from mlx_rs_amd import capi
    return capi.tile_rule(capi.Config(H, E, k, I, bits, 64, 0), T)


def kernels_with_rows(plan, counts, T, tiled, tmr):
    """The variants of `plan` (names in launch order: gate/up product, then down product; per product the
    tile classes that can occur, then the streaming kernel) that find rows in the realised routing
    `counts` (rows per expert)."""
    classes = [c for c in (0, 1, 2) if (c == 0 and T > 128) or (c == 1 and T > 64) or c == 2]
    has = {0: False, 1: False, 2: False, "streamed": False}
    from mlx_rs_amd import capi
    for c in counts:
        rows = capi.segment_rows_by_kernel(c, tiled, tmr)
        for key, n in zip((0, 1, 2, "streamed"), rows):
            if n:
                has[key] = True
    names, product = set(), []
    for n in plan:
        product.append(n)
        if n.startswith("qmm_small"):
            larges = product[:-1]
            assert len(larges) in (0, len(classes)), (plan, classes)
            for name, c in zip(larges, classes):
                if has[c]:
                    names.add(name)
            if has["streamed"]:
                names.add(n)
            product = []
    return names
