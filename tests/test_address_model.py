"""Host-side model of every global address the kernels form, checked against the buffers the C ABI hands them.

The kernels' addresses depend on shapes, launch plan and pointers only, never on operand contents, so their index
arithmetic can be restated on the CPU (numpy, one array element per lane) and every access asserted to lie inside its
operand: the prepared weight, B (or its padded copy), C / D, the K-split partial sums. The model follows
onebitsparsemul_amd/csrc/onebit_kernels.hip statement by statement (prepare_kernel, skinny_kernel with its five
B staging modes, gemm_kernel's asynchronous copy pattern and epilogue ranges, splitk_reduce_kernel, pad_b_kernel) and
takes the launch plan from the library itself (onebit_sparse_describe_launch, host-only). It covers the benchmark
configurations and the long-K shapes with 33 to 64 columns (8192 x 28672 with n = 40, 48, 64). No GPU is touched.
"""
import numpy as np
import pytest

from onebitsparsemul_amd import _native

BLOCK, SIGN_OFF, CHUNK_K, ROW_BLOCK, STAGE_K, STAGES = 1536, 1024, 256, 32, 64, 4
LANE = np.arange(64, dtype=np.int64)

# TileConfig code -> (WM, WN, FM, FN, KG), as in launch_gemm_pass
TILES = {0: (4, 1, 4, 4, 1), 1: (4, 1, 2, 4, 1), 2: (4, 1, 1, 4, 1), 3: (2, 2, 4, 4, 1), 4: (2, 2, 4, 2, 1),
         5: (2, 2, 8, 2, 1), 6: (2, 2, 2, 2, 1), 7: (2, 2, 4, 1, 1), 8: (2, 4, 4, 2, 1), 9: (4, 2, 4, 2, 1),
         10: (4, 2, 2, 2, 1), 11: (2, 4, 2, 1, 1), 12: (2, 2, 1, 2, 1), 13: (2, 2, 2, 2, 2), 14: (2, 2, 1, 2, 2),
         15: (4, 1, 4, 4, 1)}  # 15: tile 0's geometry on the 16x16x64 SMFMAC (same copies, same result region)


def prepared_bytes(m, k):
    return ((m + 31) // 32) * ((k + 255) // 256) * BLOCK


def inside(offsets, width, size, what):
    offsets = np.asarray(offsets, dtype=np.int64)
    assert offsets.size == 0 or (offsets.min() >= 0 and offsets.max() + width <= size), \
        f"{what}: [{offsets.min()}, {offsets.max() + width}) outside a buffer of {size} bytes"


def meta_offset_reference(r, c, m):
    b0, b1, b2, b345 = r & 1, (r >> 1) & 1, (r >> 2) & 1, (r >> 3) & 7
    return (c >> 1) * 2 * m + (r >> 6) * 128 + ((b1 << 6) | (b345 << 3) | (b0 << 2) | ((c & 1) << 1) | b2)


# ---------------------------------------------------------------------------------------------------------------
def check_prepare(m, k):
    kc_total, rb_total, ncols = (k + 255) // 256, m // 32, k // 16
    a_bytes, e_elems = m * k // 16, m * ncols
    i, ga = LANE & 31, LANE >> 5
    for kc in {0, kc_total // 2, kc_total - 1}:
        for rb in {0, rb_total // 2, rb_total - 1}:
            for half in (0, 1):
                j = kc * 128 + LANE + 64 * half
                ok = j < k // 2
                inside(((rb * ROW_BLOCK + j[ok] * m) >> 3), 4, a_bytes, "prepare: value bits")
            r, c0 = rb * ROW_BLOCK + i, kc * 16 + ga
            off = meta_offset_reference(r, c0, m)
            for s in range(8):
                c = c0 + 2 * s
                ok = c < ncols
                assert np.array_equal(off[ok], meta_offset_reference(r[ok], c[ok], m))  # the running offset is the closed form
                inside(off[ok] * 2, 2, e_elems * 2, "prepare: metadata")
                off = off + 2 * m
            block = (rb * kc_total + kc) * BLOCK
            inside(block + LANE * 16, 16, prepared_bytes(m, k), "prepare: block metadata")
            inside(block + SIGN_OFF + LANE * 8, 8, prepared_bytes(m, k), "prepare: block signs")


# ---------------------------------------------------------------------------------------------------------------
def skinny_variant(n, rows, b_aligned=True, tokens=False):
    nw, r = {32: (16, 1), 64: (8, 2), 128: (8, 4)}[rows]
    nc = 64 if n > 32 else 32 if n > 16 else 16
    if nc == 64:
        r = min(r, 2)
    if tokens:
        mode = "tokens"
    elif n == 1 and b_aligned:
        mode = "tokens"   # a k x 1 B is a token-major x of one token
    elif n in (2, 4) and b_aligned:
        mode = "run"      # a chunk's 256 rows as one run of 16-byte pieces
    elif n == nc and b_aligned:
        mode = "full"
    elif nc > 16 and n % 8 == 0 and b_aligned:
        mode = "b8"
    elif nc == 16 and n == 8 and b_aligned:
        mode = "b8"
    elif nc == 16 and n == 4:
        mode = "b4"
    else:
        mode = "scalar"
    return nw, r, nc, mode


def check_skinny(m, n, k, rows, tokens=False, b_aligned=True, d_size=2, splits=1):
    nw, R, nc, mode = skinny_variant(n, rows, b_aligned, tokens)
    kc_total, rb_total = (k + 255) // 256, m // 32
    img_rows = 8192 // (nc * 2)
    sub = CHUNK_K // img_rows
    prep_size, b_size = prepared_bytes(m, k), k * n * 2
    grid = (rb_total + R - 1) // R
    prefetch_b = nw <= 8 and mode != "scalar"
    cps = (kc_total + splits - 1) // splits if splits > 1 else kc_total
    splits = (kc_total + cps - 1) // cps
    assert (splits - 1) * cps < kc_total  # the launcher's check: no empty split
    b_fits = b_size < (1 << 32)
    if mode == "tokens":
        assert k * 64 * 2 < 0xFFFFFF00  # the launcher's check
    if mode == "run":
        assert k * n * 2 < 0xFFFFFF00   # the launcher's check
    for wg, split in [(g, sp) for g in sorted({0, 1, grid // 2, grid - 1} & set(range(grid)))
                      for sp in sorted({0, splits // 2, splits - 1})]:
        rb_first = wg * R
        kc_begin = split * cps
        kc_end = min(kc_begin + cps, kc_total)
        short_k = nw <= 8 and sub == 1 and mode != "scalar" and kc_end - kc_begin <= 2 * nw
        for wave in range(nw):
            first = kc_begin + wave
            # --- prepared operand through one descriptor per row block
            chunks = []
            if short_k:
                chunks += [first, first + nw]
            else:
                chunks.append(first)   # requested before the loop (clamped to the last chunk when past it)
                kc = first
                while kc < kc_end:
                    if kc + nw < kc_end:
                        chunks.append(kc + nw)
                    kc += nw
            for r in range(R):
                rb = min(rb_first + r, rb_total - 1)
                base, size = rb * kc_total * BLOCK, kc_total * BLOCK
                assert size < (1 << 32)
                for kc in chunks:
                    block = min(kc, kc_total - 1) * BLOCK
                    for off, width in ((LANE * 16, 16), (SIGN_OFF + LANE * 8, 8)):
                        inside(block + off, width, size, "split-K kernel: prepared block inside its descriptor")
                        inside(base + block + off, width, prep_size, "split-K kernel: prepared operand")
            # --- B images
            k_bases = []
            if short_k:
                k_bases += [first * CHUNK_K, (first + nw) * CHUNK_K]
            else:
                kc = first
                if prefetch_b:
                    k_bases.append(first * CHUNK_K)
                while kc < kc_end:
                    for s in range(sub):
                        k_bases.append(kc * CHUNK_K + s * img_rows)
                    if prefetch_b and kc + nw < kc_end:
                        k_bases.append(kc * CHUNK_K + nw * CHUNK_K)  # the next chunk's first image
                    kc += nw
            for k_base in k_bases:
                rows_valid = min(max(k - k_base, 0), img_rows)
                if mode == "tokens":
                    # raw buffer loads: the descriptor (n * k * 2 bytes) checks the lane offset alone and returns zero
                    # without an access when it is out of range; the scalar offset is added afterwards
                    ppt = img_rows // 8
                    tpi = 64 // ppt
                    piece_lane, token_lane = LANE % ppt, LANE // ppt
                    for i in range(8):
                        if tpi * i >= n:
                            continue  # token groups past the last token are not requested
                        if k_base + img_rows <= k:
                            lane_off = (token_lane * k + 8 * piece_lane) * 2 + i * tpi * k * 2
                            scalar_off = k_base * 2
                        else:
                            ins = k_base + 8 * piece_lane < k
                            lane_off = np.where(ins, (token_lane * k + 8 * piece_lane) * 2 + k_base * 2 + i * tpi * k * 2,
                                                0xFFFFFF00)
                            scalar_off = 0
                        assert lane_off.max() < (1 << 32)
                        accessed = lane_off + 16 <= b_size
                        assert np.array_equal(accessed, (token_lane + tpi * i < n) & (lane_off != 0xFFFFFF00))
                        inside(lane_off[accessed] + scalar_off, 16, b_size, "split-K kernel: x rows")
                    continue
                q_all = LANE[None, :] + 64 * np.arange(8)[:, None]
                if mode == "run":
                    # raw buffer loads of 16-byte pieces q = lane + 64 i < 32 n of the run that starts at k_base * n * 2
                    pieces = 32 * n
                    for i in range(2):
                        if 64 * i >= pieces:
                            continue
                        at = LANE * 16 + 1024 * i
                        if k_base + img_rows <= k:
                            lane_off = np.where(LANE + 64 * i < pieces, at, 0xFFFFFF00)
                            scalar_off = k_base * n * 2
                        else:
                            valid_bytes = rows_valid * n * 2
                            assert valid_bytes % 16 == 0  # K is a multiple of 32: no piece straddles the end of B
                            lane_off = np.where(at + 16 <= valid_bytes, k_base * n * 2 + at, 0xFFFFFF00)
                            scalar_off = 0
                        accessed = lane_off + 16 <= b_size  # the descriptor's range check looks at the lane offset alone
                        assert not accessed[lane_off == 0xFFFFFF00].any()
                        inside(lane_off[accessed] + scalar_off, 16, b_size, "split-K kernel: B run pieces")
                    continue
                if mode == "full":
                    if b_fits and k_base + img_rows <= k:
                        inside(k_base * nc * 2 + LANE[None, :] * 16 + 1024 * np.arange(8)[:, None], 16, b_size,
                               "split-K kernel: whole B image")
                    else:
                        ppr = nc // 8
                        ok = (q_all // ppr) < rows_valid
                        inside((k_base * nc + q_all[ok] * 8) * 2, 16, b_size, "split-K kernel: B image pieces")
                elif mode == "b8":
                    ppr = nc // 8
                    row, h = q_all // ppr, q_all % ppr
                    use = (row < rows_valid) & (8 * h < n)
                    inside(((k_base + row[use]) * n + 8 * h[use]) * 2, 16, b_size, "split-K kernel: padded B pieces")
                elif mode == "b4":
                    ppr = nc // 8
                    row, h = q_all // ppr, q_all % ppr
                    use = (row < rows_valid) & (h == 0)
                    inside((k_base + row[use]) * 8, 8, b_size, "split-K kernel: 8-byte B rows")
                else:  # element copies
                    valid = rows_valid * n
                    e = np.arange(img_rows * n)
                    inside((k_base * n + e[e < valid]) * 2, 2, b_size, "split-K kernel: B elements")
        # --- result: rows of the workgroup's row blocks, columns below n
        rows_out = np.arange(rb_first * 32, min((rb_first + R) * 32, m))
        cols = np.arange(n)
        elem = 4 if splits > 1 else d_size          # a split writes fp32 partial sums to its slice of the workspace
        slice0 = split * m * n * elem if splits > 1 else 0
        total = splits * m * n * elem
        if mode == "tokens":  # (one column: the same element in both layouts)
            inside(slice0 + (cols[None, :] * m + rows_out[:, None]) * elem, elem, total, "split-K kernel: y")
        else:
            inside(slice0 + (rows_out[:, None] * n + cols[None, :]) * elem, elem, total, "split-K kernel: D")
    if splits > 1:
        check_reduce(m, n, splits, d_size)


def check_reduce(m, n, splits, d_size):
    """splitk_reduce_kernel: one thread per 4 (or 1) results"""
    total = m * n
    vec = 4 if total % 4 == 0 else 1
    first = (np.arange((total // vec + 255) // 256 * 256, dtype=np.int64)) * vec
    first = first[first < total]
    for s in (0, splits - 1):
        inside((s * total + first) * 4, 4 * vec, splits * total * 4, "reduce: partial sums")
    inside(first * d_size, d_size * vec, total * d_size, "reduce: result")


# ---------------------------------------------------------------------------------------------------------------
def tile_of_block(b, tiles_m, tiles_n, group_m, xcds=8):
    total = tiles_m * tiles_n
    per, rem = total // xcds, total % xcds
    x, local = b % xcds, b // xcds
    v = x * per + min(x, rem) + local
    strip = v // (tiles_m * 4)
    strip_w = min(tiles_n - strip * 4, 4)
    w = v - strip * 4 * tiles_m
    group = w // (group_m * strip_w)
    group_h = min(tiles_m - group * group_m, group_m)
    u = w - group * group_m * strip_w
    return group * group_m + u % group_h, strip * 4 + u // group_h


def check_gemm(m, n, k, tile, splits, pad_b, tokens=False, b_aligned=True, d_size=2):
    WM, WN, FM, FN, KG = TILES[tile]
    aligned = tokens or pad_b or (n % 8 == 0 and b_aligned)
    if not aligned:
        WM, WN, FM, FN, KG = 4, 1, 1, 4, 1  # the element-copy variant
    BM, BN, NW = WM * FM * 32, WN * FN * 32, WM * WN * KG
    CH = BN // 8
    NL = STAGE_K * CH // (64 * NW)
    NA = ((BM // 32) * BLOCK + 1024 * NW - 1) // (1024 * NW)
    tiles_m, tiles_n = (m + BM - 1) // BM, (n + BN - 1) // BN
    chunks_total = (k + 255) // 256
    prep_size = prepared_bytes(m, k)
    assert prep_size < (1 << 32)  # 32-bit copy offsets (the C ABI refuses larger weights)
    cps = (chunks_total + splits - 1) // splits
    splits = (chunks_total + cps - 1) // cps
    assert (splits - 1) * cps < chunks_total  # the launcher's check: no empty split
    ldb = k if tokens else ((n + 7) // 8 * 8 if pad_b else n)
    b_size = (n * k if tokens else k * ldb) * 2
    if tokens:
        assert k * 256 * 2 < (1 << 32)
    # the workgroup -> tile mapping is a bijection
    # (for every XCD count the launcher can derive: 8 on a whole GPU, fewer on a partition)
    for xcds in (8, 4, 2, 1):
        seen = {tile_of_block(b, tiles_m, tiles_n, 8 if NW == 8 or FM * FN > 8 else 16, xcds) for b in range(tiles_m * tiles_n)}
        assert seen == {(tm, tn) for tm in range(tiles_m) for tn in range(tiles_n)}
    rb_total = m // 32
    corner_tiles = {(0, 0), (tiles_m - 1, 0), (0, tiles_n - 1), (tiles_m - 1, tiles_n - 1), (tiles_m // 2, tiles_n // 2)}
    for split in sorted({0, splits - 1, splits // 2}):
        chunk_begin = split * cps
        chunk_end = min(chunk_begin + cps, chunks_total)
        for tile_m, tile_n in corner_tiles:
            n0 = tile_n * BN
            if aligned:
                for wave in range(NW):
                    for i in range(NL):
                        slot = (NW * i + wave) * 64 + LANE
                        if tokens:
                            token = slot // 8
                            sw = np.where(True, (token >> 1) & 7, 0)
                            lc = (slot % 8) ^ sw
                            token = np.where(n0 + token >= n, 0, token)
                            b_off = (token * k + 8 * lc) * 2
                            copy_row = 8 * lc
                            stage_stride, stage0 = STAGE_K * 2, n0 * k * 2
                        else:
                            row, pc = slot // CH, slot % CH
                            sw = (((row & 3) << 2) | (((row >> 3) & 1) << 1)) if BN >= 128 else (((row >> 1) & 1) << 2)
                            lc = pc ^ sw
                            col = np.where(n0 + 8 * lc >= ldb, 0, 8 * lc)
                            b_off = (row * ldb + col) * 2
                            copy_row = row
                            stage_stride, stage0 = STAGE_K * ldb * 2, n0 * 2
                        assert b_off.max() < (1 << 32)
                        # stages copied: the first four of the split's range, then four more per chunk of the loop
                        for stage in range(chunk_begin * STAGES, chunk_end * STAGES + STAGES):
                            next_k0 = stage * STAGE_K
                            base = stage0 + stage * stage_stride
                            if next_k0 + STAGE_K <= k:
                                inside(base + b_off, 16, b_size, "main kernel: B stage copy")
                            else:
                                real = next_k0 + copy_row < k  # the other lanes copy from the block of zeros
                                inside(base + b_off[real], 16, b_size, "main kernel: B stage copy (K tail)")
                    rb0 = tile_m * (BM // 32)
                    for j in range(NA):
                        byte = (NW * j + wave) * 1024 + LANE * 16
                        blk, off = byte // BLOCK, byte % BLOCK
                        blk = np.where(blk >= BM // 32, 0, blk)
                        rb = np.minimum(rb0 + blk, rb_total - 1)
                        a_off = rb * chunks_total * BLOCK + off
                        # the chunk pointer advances while next_chunk + 1 < chunks: it never passes the last chunk
                        for chunk in range(chunk_begin, min(chunk_end + 1, chunks_total)):
                            inside(chunk * BLOCK + a_off, 16, prep_size, "main kernel: prepared block copy")
            else:
                rows_k = np.arange(k)
                cols = n0 + np.arange(BN)
                cols = cols[cols < n]
                inside((rows_k[:, None] * n + cols[None, :]) * 2, 2, k * n * 2, "main kernel: B elements")
                for fm in range(FM):
                    for wm in range(WM):
                        rb = min((tile_m * BM + wm * FM * 32) // 32 + fm, rb_total - 1)
                        for chunk in range(chunk_begin, chunk_end):
                            base = rb * chunks_total * BLOCK + chunk * BLOCK
                            inside(base + LANE * 16, 16, prep_size, "main kernel: prepared block (direct)")
                            inside(base + SIGN_OFF + LANE * 8, 8, prep_size, "main kernel: prepared signs (direct)")
            # result range of the tile: rows below m, columns below n, in this split's slice when K is split
            rows_out = np.arange(tile_m * BM, min((tile_m + 1) * BM, m))
            cols_out = np.arange(n0, min(n0 + BN, n))
            elem = 4 if splits > 1 else d_size
            slice0 = split * m * n * elem if splits > 1 else 0
            total = (splits if splits > 1 else 1) * m * n * elem
            if tokens:
                inside(slice0 + (cols_out[None, :] * m + rows_out[:, None]) * elem, elem, total, "main kernel: y")
            else:
                inside(slice0 + (rows_out[:, None] * n + cols_out[None, :]) * elem, elem, total, "main kernel: D")
    if splits > 1:
        check_reduce(m, n, splits, d_size)
    if pad_b:  # pad_b_kernel: one thread per 16-byte piece of the padded copy
        pieces_per_row = ldb // 8
        piece = np.arange(k * pieces_per_row, dtype=np.int64)
        row, col0 = piece // pieces_per_row, (piece % pieces_per_row) * 8
        for j in (0, 7):
            ok = col0 + j < n
            inside((row[ok] * n + col0[ok] + j) * 2, 2, k * n * 2, "pad_b: source")
        inside((row * ldb + col0) * 2, 16, k * ldb * 2, "pad_b: destination")


def check_call(m, n, k, tokens=False, b_aligned=True):
    plan = _native.describe_launch(m, n, k, b_aligned=b_aligned or tokens)
    if plan["kernel"] == "skinny_kernel":
        check_skinny(m, n, k, plan["rows"], tokens=tokens, b_aligned=b_aligned, splits=plan["splits"])
    else:
        check_gemm(m, n, k, plan["tile"], plan["splits"], plan["pad_b"] and not tokens, tokens=tokens, b_aligned=b_aligned)
    return plan


@pytest.fixture()
def hooks():
    def reset():
        _native.set_tile_config(-1)
        _native.set_skinny_enabled(True)
        _native.set_skinny_rows(-1)
        _native.set_split_k(-1)
        _native.set_pad_b(True)
    reset()
    yield
    reset()


@pytest.mark.parametrize("m,k", [(64, 32), (512, 512), (8192, 8192), (11008, 4096), (4096, 11008), (8192, 28672), (25600, 25600)])
def test_prepare_kernel_addresses(m, k):
    check_prepare(m, k)


@pytest.mark.parametrize("n", [40, 48, 64])
@pytest.mark.parametrize("rows,skinny", [(32, True), (64, True), (-1, False)])
def test_long_k_wide_skinny_shapes(hooks, n, rows, skinny):
    """8192 x 28672 with 33 to 64 columns: the 64-column images of the split-K kernel with 32- and 64-row workgroups, and
    the main kernel with the K split its plan chooses, plain and token-major."""
    m, k = 8192, 28672
    _native.set_skinny_rows(rows)
    _native.set_skinny_enabled(skinny)
    for tokens in (False, True):
        plan = check_call(m, n, k, tokens=tokens)
        assert (plan["kernel"] == "skinny_kernel") == skinny


@pytest.mark.parametrize("m,n,k", [(512, 512, 512), (1024, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 4096), (8192, 8192, 8192),
                                   (11008, 1, 4096), (11008, 4, 4096), (11008, 16, 4096), (4096, 1, 11008),
                                   (4096, 4, 11008), (4096, 16, 11008), (4096, 2048, 4096), (16384, 16384, 16384),
                                   (25600, 25600, 25600)])
def test_benchmark_configurations(hooks, m, n, k):
    check_call(m, n, k)
    if n >= 16:
        check_call(m, n, k, tokens=True)


@pytest.mark.parametrize("m,n,k,b_aligned", [(64, 1, 32, True), (192, 5, 800, True), (320, 8, 4128, True), (128, 13, 12320, True),
                                             (320, 17, 4128, True), (1088, 31, 2208, True), (64, 33, 32, True),
                                             (1088, 63, 2208, True), (2048, 32, 20480, True), (4096, 16, 16384, True),
                                             (576, 200, 352, True), (640, 1001, 160, True), (4096, 1001, 4096, True),
                                             (256, 264, 512, False), (1024, 203, 4128, True), (128, 1000, 4128, True),
                                             (28672, 40, 512, True), (20480, 64, 1024, True), (4096, 384, 11008, True),
                                             (64, 72, 64, False), (2112, 1032, 64, True), (4096, 16, 16384, True),
                                             (2048, 33, 28672, True), (11008, 32, 28672, True), (192, 5, 12320, True),
                                             (320, 2, 4128, True), (320, 4, 4128, True), (2240, 1, 8224, True),
                                             (192, 4, 800, False), (192, 2, 12320, True)])
def test_ragged_and_split_shapes(hooks, m, n, k, b_aligned):
    for rows in (-1, 32, 64, 128):
        _native.set_skinny_rows(rows)
        check_call(m, n, k, b_aligned=b_aligned)
    _native.set_skinny_rows(-1)
    check_call(m, n, k, tokens=True)
    for splits in (2, 3, 16):  # the split-K kernel's own K split over workgroups (n <= 64), forced
        _native.set_split_k(splits)
        for rows in (32, 64, 128):
            _native.set_skinny_rows(rows)
            check_call(m, n, k, b_aligned=b_aligned)
            check_call(m, n, k, tokens=True)
    _native.set_skinny_rows(-1)
    _native.set_skinny_enabled(False)
    for splits in (-1, 1, 3, 16):
        _native.set_split_k(splits)
        check_call(m, n, k, b_aligned=b_aligned)
        check_call(m, n, k, tokens=True)


@pytest.mark.parametrize("tile", sorted(TILES))
def test_every_tile_configuration(hooks, tile):
    _native.set_tile_config(tile)
    _native.set_skinny_enabled(False)
    for m, n, k in ((1024, 512, 1024), (576, 264, 192), (2112, 1032, 64), (8192, 8192, 8192)):
        check_call(m, n, k)
        if tile in (4, 6, 9, 10, 11, 12, 13, 14, 15):
            check_call(m, n, k, tokens=True)


def test_the_model_catches_an_out_of_range_access():
    """the checker itself: a prepared operand one block too small, or B one row too short, must be flagged"""
    with pytest.raises(AssertionError):
        inside(np.array([0, prepared_bytes(64, 256) - 8]), 16, prepared_bytes(64, 256), "probe")
    real = prepared_bytes

    def short(m, k):
        return real(m, k) - BLOCK
    globals()["prepared_bytes"] = short
    try:
        with pytest.raises(AssertionError):
            check_skinny(1024, 16, 4096, 64)
        with pytest.raises(AssertionError):
            check_gemm(1024, 512, 1024, 9, 1, False)
    finally:
        globals()["prepared_bytes"] = real


# ---- the epilogue's turn through the LDS scratch (gemm_kernel, coalesced form) ------------------------------------
# Restates the index arithmetic of the two forms: fp32 rows [32][WCOLS] and packed fp16 row pairs [16][WCOLS], both with
# the column swizzle (16-byte slots swapped in pairs on odd lines, 128-byte halves swapped when bit 2 of the row / bit 1
# of the row pair is set and a line has at least 64 columns).

def _half_swap(wcols):
    return 32 if wcols >= 64 else 0


def _scratch_rows_model(fn_count):
    """(writes, reads) of the fp32 form for one 32-row block: dicts word -> (row, column) written / read."""
    wcols = fn_count * 32
    writes, reads = {}, {}
    for lane in range(64):
        col_lane, row_lane = lane & 31, 4 * (lane >> 5)
        half_write = (lane >> 5) * _half_swap(wcols)
        for fn in range(fn_count):
            for v in range(16):
                row = 8 * (v // 4) + row_lane + v % 4
                word = row * wcols + ((fn * 32 + col_lane) ^ half_write ^ ((v & 1) << 2))
                assert word not in writes
                writes[word] = (row, fn * 32 + col_lane)
    per_row = wcols // 8
    for it in range(32 * per_row // 64):
        for lane in range(64):
            piece = it * 64 + lane
            r, c8 = piece // per_row, (piece % per_row) * 8
            sw = ((r & 1) << 2) ^ (((r >> 2) & 1) * _half_swap(wcols))
            for part, base in ((0, c8), (1, c8 + 4)):
                for j in range(4):
                    reads[r * wcols + (base ^ sw) + j] = (r, base + j)
    return wcols, writes, reads


def _scratch_pairs_model(fn_count):
    """the packed form: word -> (row pair, column)."""
    wcols = fn_count * 32
    writes, reads = {}, {}
    for lane in range(64):
        col_lane, row_lane = lane & 31, 4 * (lane >> 5)
        half_write = (lane >> 5) * _half_swap(wcols)
        for fn in range(fn_count):
            for q in range(8):
                pair = 4 * (q // 2) + (row_lane >> 1) + (q & 1)
                rows = 8 * (q // 2) + row_lane + 2 * (q % 2)   # registers 2q, 2q + 1 of the accumulator layout
                assert rows == 2 * pair
                word = pair * wcols + ((fn * 32 + col_lane) ^ half_write ^ ((q & 1) << 2))
                assert word not in writes
                writes[word] = (pair, fn * 32 + col_lane)
    per_pair = wcols // 8
    tasks = 16 * per_pair
    for it in range((tasks + 63) // 64):
        for lane in range(64):
            task = it * 64 + lane
            if task >= tasks:
                continue
            pair, c8 = task // per_pair, (task % per_pair) * 8
            sw = ((pair & 1) << 2) ^ (((pair >> 1) & 1) * _half_swap(wcols))
            for base in (c8, c8 + 4):
                for j in range(4):
                    reads[pair * wcols + (base ^ sw) + j] = (pair, base + j)
    return wcols, writes, reads


@pytest.mark.parametrize("fn_count", [1, 2, 4])
@pytest.mark.parametrize("model,lines", [(_scratch_rows_model, 32), (_scratch_pairs_model, 16)])
def test_epilogue_scratch_is_written_once_and_read_back_where_it_was_written(model, lines, fn_count):
    wcols, writes, reads = model(fn_count)
    assert sorted(writes) == list(range(lines * wcols))          # every word of the wavefront's scratch, once, in range
    assert reads == writes                                       # a reader finds (line, column) where the writer put it


def test_epilogue_scratch_swizzle_avoids_bank_conflicts():
    # The tiles the planner uses have 64-column wavefront tiles. 64 banks of 4 bytes. A 4-byte store instruction: the 32
    # lanes of each half-wavefront touch 32 different banks and the two halves touch different ones. A 16-byte read: the
    # 16 lanes served together (two lines) touch 64 different banks.
    wcols = 64
    for v in range(16):
        banks = []
        for lane in range(64):
            row = 8 * (v // 4) + 4 * (lane >> 5) + v % 4
            word = row * wcols + ((lane & 31) ^ ((lane >> 5) * 32) ^ ((v & 1) << 2))
            banks.append(word % 64)
        assert len(set(banks)) == 64
    per_row = wcols // 8
    for group in range(4):
        banks = []
        for lane in range(16 * group, 16 * group + 16):
            r, c8 = lane // per_row, (lane % per_row) * 8
            sw = ((r & 1) << 2) ^ (((r >> 2) & 1) * 32)
            banks += [(r * wcols + (c8 ^ sw) + j) % 64 for j in range(4)]
        assert len(set(banks)) == 64


# ---------------------------------------------------------------------------------------------------------------
# the split-K kernel's 16x16x64 form: which K positions of a chunk each lane group of an instruction multiplies, on
# the A side (prepared block lanes after v_permlane16_swap) and on the B side (rows of the image a lane reads)
# ---------------------------------------------------------------------------------------------------------------
def _permlane16_swap(x, y):
    """v_permlane16_swap x, y: the odd 16-lane rows of x trade places with the even rows of y"""
    x, y = x.copy(), y.copy()
    for row in (0, 2):
        lo, hi = slice(16 * row, 16 * row + 16), slice(16 * (row + 1), 16 * (row + 2))
        x[hi], y[lo] = y[lo].copy(), x[hi].copy()
    return x, y


def test_split_k_16x16x64_operands_agree_on_k():
    lane = np.arange(64)
    # lane of the prepared block: row lane % 32, half ga = lane // 32 of each 32-wide K step; metadata register d
    # holds steps 2 d (low half word, ABID 0) and 2 d + 1 (high, ABID 1); the value tracked here is (lane, register)
    src = {d: lane * 8 + d for d in range(4)}
    for P in range(2):
        first, second = _permlane16_swap(src[2 * P], src[2 * P + 1])
        for half, reg in enumerate((first, second)):          # operands of block rows 0-15 and 16-31
            src_lane, src_reg = reg // 8, reg % 8
            assert np.array_equal(src_lane % 32, 16 * half + lane % 16)  # every lane group holds its own row l % 16
            ga = src_lane // 32
            for abid in range(2):
                step = 2 * src_reg + abid
                a_first_k = 32 * step + 16 * ga            # the lane's 16 consecutive K positions of the chunk
                # the instruction pairs A group g, position j with B group (16 g + j) % 32 // 8, slot
                # 8 ((16 g + j) // 32) + (16 g + j) % 8; a B lane of group gb reads image rows
                # base + {0..7} (slots 0-7) and base + 16 + {0..7} (slots 8-15)
                for g in range(4):
                    first_k = a_first_k[16 * g]
                    assert (a_first_k[16 * g:16 * g + 16] == first_k).all()
                    for j in range(16):
                        ik = 16 * g + j
                        gb, slot = (ik % 32) // 8, 8 * (ik // 32) + ik % 8
                        base = 128 * P + 32 * abid + 64 * (gb >> 1) + 8 * (gb & 1)
                        assert base + slot % 8 + 16 * (slot // 8) == first_k + j
                # sign bits: register q of step s uses shift 4 (s % 4) + q of the lane's word for steps 4 P ... 4 P + 3;
                # the kernel shifts by 8 (g % 2) once and then by 4 abid + q
                g_of_lane = lane // 16
                assert np.array_equal(4 * (step % 4), 8 * (g_of_lane % 2) + 4 * abid)
                assert (step // 4 == P).all()
    # the sign words travel like the metadata: a register swapped with its own copy puts the word of block lane
    # (row, ga) in lane groups g = 2 ga and 2 ga + 1 of the half that holds the row
    first, second = _permlane16_swap(lane.copy(), lane.copy())
    for half, reg in enumerate((first, second)):
        assert np.array_equal(reg % 32, 16 * half + lane % 16)
        assert np.array_equal(reg // 32, lane // 32)
