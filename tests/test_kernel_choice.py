"""The kernel-choice functions of the library, walked over grids of shapes on the CPU (decx_hip_sgemm_plan,
decx_hip_hgemm_plan: host-only entry points that run the very functions decx_hip_sgemm / decx_hip_hgemm_f32acc choose
their kernel with; no device call, 256 compute units assumed before decx_hip_init).

What is pinned: every answer is a kernel the dispatch builds for that kind of operand; operands the vector loaders cannot
take get the element-wise loader; a pitch of 2^21 floats or more never reaches the fp32 tiles that address a tile's rows
with 32-bit byte offsets (18 - 28), nor does a pitch beyond the fp16 limits reach the fp16 vector kernels; a forced
variant is honoured only where it can run; every automatic split over K fits the workspace decx_hip_init reserves."""
import ctypes
import itertools

import pytest

from backup_1_amd import capi

SIZES = [1, 7, 16, 31, 64, 100, 128, 200, 256, 500, 512, 1000, 1024, 1500, 2048, 3000, 4096, 4500, 8192]
FP32_TILES = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 14, 15, 16}          # register-staged tiles the dense dispatch builds
FP32_CHAINS = {11, 12, 13, 23}                                     # one wave per block
FP32_DMA = {18, 19, 20, 21, 22, 24, 25, 26, 27, 28}                # LDS-DMA tiles: 32-bit byte offsets inside a tile
FP16_BUILT = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 15, 16, 17}
DMA_MAX_PITCH = 1 << 21
RESERVED_WORKSPACE = 2 * 256 * 128 * 128 * 4                       # what decx_hip_init reserves on 256 CUs


def pad(x, unit):
    return (x + unit - 1) // unit * unit


@pytest.fixture
def lib():
    L = capi.lib()
    prev32, prev16 = L.decx_hip_set_sgemm_variant(0), L.decx_hip_set_hgemm_variant(0)
    yield L
    L.decx_hip_set_sgemm_variant(prev32)
    L.decx_hip_set_hgemm_variant(prev16)


def test_fp32_choice_over_a_grid_of_shapes(lib):
    seen = set()
    for M, N, K in itertools.product(SIZES, repeat=3):
        for batch in (1, 3):
            lda, ldb = pad(K, 8), pad(N, 8)
            v = lib.decx_hip_sgemm_plan(M, N, K, batch, lda, ldb, 1)
            assert v in FP32_TILES | FP32_CHAINS | FP32_DMA, (M, N, K, batch, v)
            assert v == lib.decx_hip_sgemm_plan(M, N, K, batch, lda, ldb, 1)
            seen.add(v)
            # pitches from which a tile's byte offsets leave 31 bits: never the LDS-DMA tiles, whichever operand it is
            for wide_a, wide_b in ((DMA_MAX_PITCH, ldb), (lda, DMA_MAX_PITCH), (DMA_MAX_PITCH + 8, DMA_MAX_PITCH + 8)):
                w = lib.decx_hip_sgemm_plan(M, N, K, batch, max(wide_a, lda), max(wide_b, ldb), 1)
                assert w in FP32_TILES | FP32_CHAINS, (M, N, K, batch, wide_a, wide_b, w)
            # just below the limit the choice is the one of ordinary pitches
            assert lib.decx_hip_sgemm_plan(M, N, K, batch, max(DMA_MAX_PITCH - 4, lda), max(DMA_MAX_PITCH - 4, ldb), 1) == v
            # operands off the 16-byte grid, or pitches not in fours: the element-wise loader
            assert lib.decx_hip_sgemm_plan(M, N, K, batch, lda, ldb, 0) == 0
            assert lib.decx_hip_sgemm_plan(M, N, K, batch, lda + 1, ldb, 1) == 0
            assert lib.decx_hip_sgemm_plan(M, N, K, batch, lda, ldb + 2, 1) == 0
    # the grid reaches every family: the big LDS-DMA tiles, the small ones, the block chains and the register-staged tiles
    assert {26, 27, 20, 24, 18, 12, 23} <= seen and seen & FP32_TILES, sorted(seen)


def test_fp32_headline_and_config_shapes(lib):
    assert lib.decx_hip_sgemm_plan(8192, 8192, 8192, 1, 8192, 8192, 1) == 26        # 256x256 LDS-DMA tile
    assert lib.decx_hip_sgemm_plan(4096, 4096, 4096, 1, 4096, 4096, 1) == 26
    assert lib.decx_hip_sgemm_plan(3000, 4500, 1500, 1, 1504, 4504, 1) == 27        # 252 tiles of 256x224
    assert lib.decx_hip_sgemm_plan(1024, 1024, 1024, 1, 1024, 1024, 1) in (18, 19)  # one 64x64 tile per CU
    assert lib.decx_hip_sgemm_plan(64, 1024, 65536, 1, 65536, 1024, 1) in FP32_CHAINS
    assert lib.decx_hip_sgemm_plan(0, 8, 8, 1, 8, 8, 1) == -1 and lib.decx_hip_sgemm_plan(8, 8, 8, 1, 4, 8, 1) == -1


def test_fp32_tall_results_take_the_tiles_that_pad_them_least(lib):
    """Many rows under at most 256 columns (the shape of a lowered convolution): the measured choices."""
    plan = lambda M, K, N: lib.decx_hip_sgemm_plan(M, N, K, 1, pad(K, 8), pad(N, 8), 1)
    assert plan(30000, 512, 48) == 18             # not the 128x128 tile, which would be 5/8 padding
    assert plan(82944, 864, 96) == 25 and plan(82944, 864, 160) == 25      # 96 = 3 x 32, 160 = 5 x 32 columns
    assert plan(409600, 576, 64) == 18 and plan(200000, 256, 64) == 18     # one 64x64 tile across
    assert plan(300000, 128, 64) == 9 and plan(400000, 32, 64) == 9        # a few K steps only: 128x64 register-staged tiles
    assert plan(147456, 1152, 128) == 20 and plan(200000, 128, 128) == 20 and plan(150000, 2048, 256) == 20
    assert plan(262144, 288, 32) == 25 and plan(150000, 2304, 32) == 25 and plan(600000, 576, 16) == 25    # tiles 32 wide
    assert plan(100000, 4096, 128) in FP32_TILES  # 782 tiles of 128x128 would be 3.05 rounds
    for N in range(1, 257):                       # every width: a kernel the dispatch builds; on a long K never a 128-wide tile that is mostly padding
        for M, K in ((100000, 128), (100000, 600), (250000, 2048)):
            v = plan(M, K, N)
            assert v in FP32_TILES | FP32_DMA, (M, K, N, v)
            assert not (K > 256 and v == 20 and N % 128 != 0 and N % 128 < 100), (M, K, N)


def split_plan(lib, M, K, N, batch=1, lda=None, ldb=None, aligned=1):
    shape, by_columns = ctypes.c_int(-1), ctypes.c_int(-1)
    first = lib.decx_hip_sgemm_plan_split(M, N, K, batch, lda or pad(K, 8), ldb or pad(N, 8), aligned, ctypes.byref(shape), ctypes.byref(by_columns))
    return first, shape.value, by_columns.value


def test_fp32_two_launch_plans_are_whole_rounds_of_a_256_row_tile(lib):
    """decx_hip_sgemm_plan_split over a grid: a first launch is whole tile rows (columns) of its tile that fit the whole
    rounds of 256 compute units and leave something for the second launch; no plan for a forced variant, a batch, a short
    K, operands the LDS-DMA tiles cannot take, or a result of whole rounds."""
    widths = {26: 256, 27: 224, 28: 192}
    planned = 0
    for M in range(1500, 9000, 293):
        for N in range(1500, 9000, 347):
            for K in (512, 1500, 4096):
                first, shape, by_columns = split_plan(lib, M, K, N)
                if first == 0:
                    assert shape == 0 and by_columns == 0
                    continue
                planned += 1
                assert shape in widths, (M, K, N, shape)
                tiles_m, tiles_n = -(-M // 256), -(-N // widths[shape])
                whole = tiles_m * tiles_n // 256
                assert whole >= 1 and tiles_m * tiles_n % 256 != 0
                if by_columns:
                    assert first % widths[shape] == 0 and 0 < first < N and first // widths[shape] * tiles_m <= whole * 256
                    assert (first // widths[shape] + 1) * tiles_m > whole * 256        # as many columns as the rounds hold
                else:
                    assert first % 256 == 0 and 0 < first < M and first // 256 * tiles_n <= whole * 256
                    assert (first // 256 + 1) * tiles_n > whole * 256
                assert split_plan(lib, M, K, N, batch=2)[0] == 0
                assert split_plan(lib, M, K, N, lda=DMA_MAX_PITCH)[0] == 0 and split_plan(lib, M, K, N, ldb=DMA_MAX_PITCH)[0] == 0
                assert split_plan(lib, M, K, N, aligned=0)[0] == 0 and split_plan(lib, M, K, N, ldb=pad(N, 8) + 2)[0] == 0
    assert planned > 100
    # the measured ones: 4352^2 is 289 tiles of 256x256 -- 15 tile rows in one round, 512 rows left
    assert split_plan(lib, 4352, 4096, 4352) == (3840, 26, 0)
    assert split_plan(lib, 4096, 4096, 4608) == (3584, 27, 1) and split_plan(lib, 2048, 4096, 6212) == (6144, 28, 1)
    for whole_rounds in ((8192, 8192, 8192), (4096, 4096, 4096), (6144, 6144, 6144), (3000, 1500, 4500), (1024, 1024, 1024)):
        assert split_plan(lib, *whole_rounds)[0] == 0
    assert split_plan(lib, 4352, 256, 4352)[0] == 0                                    # short K
    for forced in (26, 7, 34):
        lib.decx_hip_set_sgemm_variant(forced)
        assert split_plan(lib, 4352, 4096, 4352)[0] == 0
    lib.decx_hip_set_sgemm_variant(34)                                                 # 34 leaves the kernel choice alone
    assert lib.decx_hip_sgemm_plan(4352, 4352, 4096, 1, 4096, 4352, 1) in FP32_TILES | FP32_DMA
    lib.decx_hip_set_sgemm_variant(0)
    assert split_plan(lib, 0, 8, 8)[0] == -1


def test_fp16_two_launch_plans_are_whole_rounds_of_the_256_tile(lib):
    def plan(M, K, N, batch=1, lda=None, ldb=None, aligned=1):
        by_columns = ctypes.c_int(-1)
        first = lib.decx_hip_hgemm_plan_split(M, N, K, batch, lda or pad(K, 16), ldb or pad(N, 16), aligned, ctypes.byref(by_columns))
        return first, by_columns.value
    planned = 0
    for M in range(1500, 9000, 293):
        for N in range(1500, 9000, 347):
            for K in (512, 4096):
                first, by_columns = plan(M, K, N)
                if first == 0:
                    continue
                planned += 1
                tiles_m, tiles_n = -(-M // 256), -(-N // 256)
                whole = tiles_m * tiles_n // 256
                assert whole >= 1 and tiles_m * tiles_n % 256 != 0 and first % 256 == 0
                lines, across, extent = first // 256, (tiles_m if by_columns else tiles_n), (N if by_columns else M)
                assert 0 < first < extent and lines * across <= whole * 256 < (lines + 1) * across
                assert plan(M, K, N, batch=2)[0] == 0 and plan(M, K, N, aligned=0)[0] == 0 and plan(M, K, N, lda=pad(K, 16) + 4)[0] == 0
    assert planned > 100
    assert plan(4352, 4096, 4352) == (3840, 0)
    for whole_rounds in ((8192, 8192, 8192), (4096, 4096, 4096), (3000, 1500, 4500), (1024, 1024, 1024), (64, 65536, 1024)):
        assert plan(*whole_rounds)[0] == 0
    assert plan(4352, 256, 4352)[0] == 0
    for forced in (15, 8, 11, 20):
        lib.decx_hip_set_hgemm_variant(forced)
        assert plan(4352, 4096, 4352)[0] == 0
    lib.decx_hip_set_hgemm_variant(20)                                                 # 20 leaves the kernel choice alone
    assert lib.decx_hip_hgemm_plan(4352, 4352, 4096, 1, 4096, 4352, 1, None) in (8, 9, 15)
    lib.decx_hip_set_hgemm_variant(0)


def test_convolution_two_launch_plans_are_whole_rounds_of_the_256_tile(lib):
    def plan(H, W, C, N, k=3, flag=1):
        shape = ctypes.c_int(-1)
        rows = lib.decx_hip_conv_plan_split(H, W, C, N, k, k, flag, ctypes.byref(shape))
        return rows, shape.value
    planned = 0
    for H in range(150, 1200, 37):
        for C in (16, 48, 64, 128, 256):
            for N in (32, 64, 128, 256, 384, 512):
                for flag in (0, 1):
                    rows, shape = plan(H, H + 3, C, N, flag=flag)
                    if rows == 0:
                        assert shape == 0
                        continue
                    planned += 1
                    Hout, Wout = (H, H + 3) if flag else (H - 2, H + 1)
                    tiles_n = -(-N // 256)
                    whole = -(-Hout * Wout // 256) * tiles_n // 256
                    assert shape == 7 and 0 < rows < Hout and whole >= 1 and 9 * C >= 512
                    assert -(-rows * Wout // 256) * tiles_n <= whole * 256          # the first launch fits the whole rounds
    assert planned > 20
    assert plan(300, 300, 128, 256) == (218, 7)                        # measured: 418 -> 383 us
    assert plan(224, 224, 64, 128)[0] == 0 and plan(512, 512, 256, 256)[0] == 0        # single round; four whole rounds
    assert plan(300, 300, 16, 256)[0] == 0                             # K = 144: short
    for forced in (7, 16, 34):
        lib.decx_hip_set_sgemm_variant(forced)
        assert plan(300, 300, 128, 256)[0] == 0
    lib.decx_hip_set_sgemm_variant(0)
    assert plan(0, 300, 128, 256)[0] == -1 and plan(2, 300, 128, 256, flag=0)[0] == -1


def test_forced_fp32_variants_stay_where_they_can_run(lib):
    for forced in sorted(FP32_TILES | FP32_CHAINS | FP32_DMA):
        lib.decx_hip_set_sgemm_variant(forced)
        for M, N, K in ((300, 200, 260), (2048, 2048, 512), (37, 4097, 24)):
            lda, ldb = pad(K, 8), pad(N, 8)
            v = lib.decx_hip_sgemm_plan(M, N, K, 1, lda, ldb, 1)
            assert v == forced, (forced, M, N, K, v)
            w = lib.decx_hip_sgemm_plan(M, N, K, 1, DMA_MAX_PITCH, DMA_MAX_PITCH, 1)
            assert (w == forced) if forced not in FP32_DMA else (w in FP32_TILES | FP32_CHAINS), (forced, w)
            assert lib.decx_hip_sgemm_plan(M, N, K, 1, lda, ldb, 0) == 0
    lib.decx_hip_set_sgemm_variant(0)


def test_fp16_choice_over_a_grid_of_shapes(lib):
    splits = ctypes.c_int(0)
    seen = set()
    for M, N, K in itertools.product(SIZES + [16384, 65536], repeat=3):
        if M * N > (1 << 28) or M * K > (1 << 30) or K * N > (1 << 30):
            continue
        for batch in (1, 3):
            lda, ldb = pad(K, 16), pad(N, 16)
            v = lib.decx_hip_hgemm_plan(M, N, K, batch, lda, ldb, 1, ctypes.byref(splits))
            assert v in {8, 9, 11, 15, 17}, (M, N, K, batch, v)                  # the automatic choices
            seen.add(v)
            if v == 17:          # the walk over several tiles: whole tiles only, more of them than CUs, the measured range of K
                assert batch == 1 and M % 256 == 0 and N % 256 == 0 and K % 128 == 0 and 128 <= K <= 3072 and (M // 256) * (N // 256) > 256
            if v == 11:
                assert batch == 1 and splits.value >= 2 and K // splits.value >= 512
                assert M * N * 4 * splits.value <= RESERVED_WORKSPACE, (M, N, K, splits.value)
            else:
                assert splits.value == 0
            assert lib.decx_hip_hgemm_plan(M, N, K, batch, lda, ldb, 0, None) == 0
            assert lib.decx_hip_hgemm_plan(M, N, K, batch, lda + 4, ldb, 1, None) == 0
    assert seen == {8, 9, 11, 15, 17}
    # a 256-row tile of A beyond 4 GiB, 64 rows of B beyond 4 GiB: the element-wise kernel, which uses 64-bit addresses
    assert lib.decx_hip_hgemm_plan(300, 260, 200, 1, 1 << 23, 272, 1, None) == 0
    assert lib.decx_hip_hgemm_plan(300, 260, 200, 1, 208, 1 << 25, 1, None) == 0
    assert lib.decx_hip_hgemm_plan(300, 260, 200, 1, 6 << 20, 6 << 20, 1, None) in {8, 9, 15}
    assert lib.decx_hip_hgemm_plan(8192, 8192, 8192, 1, 8192, 8192, 1, None) == 15


def test_forced_fp16_variants(lib):
    splits = ctypes.c_int(0)
    for forced in sorted(FP16_BUILT - {11}):
        lib.decx_hip_set_hgemm_variant(forced)
        assert lib.decx_hip_hgemm_plan(64, 1024, 65536, 1, 65536, 1024, 1, ctypes.byref(splits)) == forced and splits.value == 0
        assert lib.decx_hip_hgemm_plan(300, 260, 200, 3, 208, 272, 1, None) == forced
        assert lib.decx_hip_hgemm_plan(300, 260, 200, 1, 208, 272, 0, None) == 0
    lib.decx_hip_set_hgemm_variant(11)                                           # forces the split where K allows one
    assert lib.decx_hip_hgemm_plan(512, 512, 4096, 1, 4096, 512, 1, ctypes.byref(splits)) == 11 and splits.value >= 2
    assert lib.decx_hip_hgemm_plan(512, 512, 512, 1, 512, 512, 1, ctypes.byref(splits)) in {8, 9, 15}
    lib.decx_hip_set_hgemm_variant(0)


def test_patch_kernels_keep_their_offsets_on_the_right_side_of_two_gib(lib):
    """src_bytes + apron + reach < 2^31, with apron = (oy row_stride + ox dpitch) e + 16 and reach = ((16 + kh) row_stride +
    (16 + kw) dpitch) e: evaluated here independently and compared around the boundary."""
    def fits(H, W, dp, rs, kh, kw, flag, e):
        src = ((H - 1) * rs + W * dp) * e
        oy, ox = (kh // 2, kw // 2) if flag else (0, 0)
        return int(src < 2 ** 31 and src + (oy * rs + ox * dp) * e + 16 + ((16 + kh) * rs + (16 + kw) * dp) * e < 2 ** 31)

    for e, dp, W in ((4, 64, 1024), (2, 64, 1024), (4, 32, 4000), (2, 256, 3000)):
        rs = W * dp
        for kh, kw, flag in ((3, 3, 1), (3, 3, 0), (7, 5, 1), (1, 1, 1)):
            h_limit = 2 ** 31 // (rs * e)                       # about where the tensor alone reaches 2 GiB
            answers = set()
            for H in range(max(1, h_limit - 40), h_limit + 3):
                got = lib.decx_hip_conv_patch_offsets_fit(H, W, dp, rs, kh, kw, flag, e)
                assert got == fits(H, W, dp, rs, kh, kw, flag, e), (H, W, dp, kh, kw, flag, e)
                answers.add(got)
            assert answers == {0, 1}                            # the sweep crosses the boundary
    assert lib.decx_hip_conv_patch_offsets_fit(224, 224, 64, 224 * 64, 3, 3, 1, 4) == 1
    assert lib.decx_hip_conv_patch_offsets_fit(224, 224, 64, 100, 3, 3, 1, 4) == -1
    assert lib.decx_hip_conv_patch_offsets_fit(224, 224, 64, 224 * 64, 3, 3, 1, 3) == -1
