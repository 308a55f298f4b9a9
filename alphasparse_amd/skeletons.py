"""The nine compressed-view graph skeletons of the white-list search
(upstream whilte_list_path_impl.cc:180-3095) as (strategy, knobs) lists + template types."""
from . import _capi as K


def skeleton(name, **kw):
    """-> (list of (strategy, knobs) for one compressed sub-matrix, list of candidate templates)."""
    if name == "S1":  # SELL: rows padded to m, BLBs of m rows, one TLB per row
        m = kw.get("m", 64)
        return ([(K.COMPRESSED_ROW_PADDING_DIRECT, (m, 1)), (K.COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY, (m,)),
                 (K.COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE, ())], [K.DIRECT_ATOM_TEMPLATE_WARP_COMPRESS])
    if name == "S5":  # ELL
        return ([(K.COMPRESSED_ROW_PADDING_DIRECT, (kw.get("wave", 64), 1)), (K.COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE, ())],
                [K.DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS])
    if name == "S9":  # CSR5-like
        return ([(K.COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT, (kw.get("t", 4),))],
                [K.UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE,
                 K.UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE])
    if name == "S4":  # CSR-vector with fixed-size row pieces
        return ([(K.COMPRESSED_WARP_LEVEL_COL_DIV_FIXED, (kw.get("c", 64),))], [K.DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE])
    if name == "S6":
        m, ln = kw.get("m", 4), kw.get("len", 1)
        return ([(K.COMPRESSED_ROW_PADDING_DIRECT, (m, ln)), (K.COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY, (m,)),
                 (K.COMPRESSED_WARP_LEVEL_COL_DIV_FIXED, (kw.get("c", 64),))], [K.SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE])
    if name == "S7":
        return ([(K.COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ, (kw.get("n", 512),)),
                 (K.COMPRESSED_WARP_LEVEL_COL_DIV_FIXED, (kw.get("c", 64),))], [K.SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE])
    if name == "S8":  # long rows cut into one-row BLBs
        return ([(K.COMPRESSED_TBLOCK_LEVEL_COL_DIV_FIXED, (kw.get("b", 1024),))], [K.SHARED_MEMORY_LONG_ROW_TEMPLATE])
    if name == "S2":
        m, ln = kw.get("m", 64), kw.get("len", 1)
        return ([(K.COMPRESSED_ROW_PADDING_DIRECT, (m, ln)), (K.COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY, (m,)),
                 (K.COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED, (kw.get("s", 4),))], [K.SHARED_MEMORY_TEMPLATE_WARP_COMPRESS])
    if name == "S3":
        return ([(K.COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ, (kw.get("n", 512),)),
                 (K.COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED, (kw.get("s", 4),))], [K.SHARED_MEMORY_TEMPLATE_WARP_COMPRESS])
    # the two general templates are outside the white list; these graphs give every WLB its own TLB size
    if name == "B1":  # BLBs of m rows, WLBs of w rows, one TLB per row
        return ([(K.COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY, (kw.get("m", 64),)),
                 (K.COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY, (kw.get("w", 16),)),
                 (K.COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE, ())], [K.DIRECT_ATOM_TEMPLATE])
    if name == "B2":  # BLBs by nnz, WLBs of w rows, rows cut into TLBs of s elements, partials reduced in LDS
        return ([(K.COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ, (kw.get("n", 512),)),
                 (K.COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY, (kw.get("w", 16),)),
                 (K.COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED, (kw.get("s", 4),))], [K.SHARED_MEMORY_TEMPLATE])
    if name == "X1":  # long rows cut at column slice boundaries, the slice of x kept in LDS (no upstream counterpart)
        return ([(K.COMPRESSED_TBLOCK_LEVEL_COL_DIV_COL_SLICE, (kw.get("slice", 32768),))], [K.SHARED_MEMORY_X_SLICE_TEMPLATE])
    if name == "T1":  # 2-D tiles (row group x column slice), slice of x and row sums kept in LDS (no upstream counterpart)
        return ([(K.COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE,
                  (kw.get("slice", 32768), kw.get("group", 8192), kw.get("b", 8192)))], [K.SHARED_MEMORY_TILE_TEMPLATE])
    if name == "T2":  # the same tiles in two passes: products to scratch, then row sums per summing group (no upstream counterpart)
        return ([(K.COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE,
                  (kw.get("slice", 32768), kw.get("group", 4096), kw.get("b", 8192)))], [K.SHARED_MEMORY_PRODUCT_BIN_TEMPLATE])
    raise ValueError("unknown skeleton " + name)


BLB_LEVEL_STRATEGIES = (K.COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY, K.COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ)


def apply_skeleton(matrix, sub, name, block_sort=None, **kw):
    """Run the skeleton's strategies on one compressed sub-matrix and complete the blocking.
    block_sort: None, or the list of BLBs whose rows are sorted by falling length right after the BLB level is
    made (COMPRESSED_BLOCK_SORT; an empty list = every BLB)."""
    strategies, templates = skeleton(name, **kw)
    for s, p in strategies:
        matrix.execute_strategy(s, sub, p)
        if block_sort is not None and s in BLB_LEVEL_STRATEGIES:
            matrix.execute_node(K.COMPRESSED_BLOCK_SORT, sub, lst=block_sort)
    matrix.complete_blocking(sub)
    return templates
