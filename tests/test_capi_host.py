"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol
include/qgemm.h declares, validates arguments before touching a device, and its tile
raster is a bijection."""
import ctypes as C
import os
import re

import pytest

import qgemm_amd as Q
from qgemm_amd import lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "qgemm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(qgemm_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = L.load_library()
    names = _declared_symbols()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/qgemm.h but not exported"
        assert n in L.SIGNATURES, f"{n} has no ctypes signature in qgemm_amd/lib.py"
    # and nothing in the binding that the header does not declare
    assert sorted(L.SIGNATURES) == names


def test_status_strings():
    lib = L.load_library()
    assert lib.qgemm_status_string(0) == b"ok"
    # the reference's throw texts, hip_mix_gemm_kernel.cpp:460,485,503
    assert b"BLOCK_TILE_SIZE_M" in lib.qgemm_status_string(6)
    assert b"BLOCK_TILE_SIZE_N" in lib.qgemm_status_string(7)
    assert b"BLOCK_TILE_SIZE_K" in lib.qgemm_status_string(8)
    assert lib.qgemm_status_string(12345) == b"unknown status"


def test_argument_validation_needs_no_device():
    lib = L.load_library()
    one = C.c_void_p(16)
    # unknown dtype / dtype pair
    assert lib.qgemm_gemm(99, 0, 1, one, 16, one, 16, one, 16, 16, 16, 16, None) == 2
    assert lib.qgemm_gemm(Q.DT_BF16, Q.DT_I32, 1, one, 16, one, 16, one, 16, 16, 16, 16, None) == 2
    # bad layout enum, leading dimension smaller than the row
    assert lib.qgemm_gemm(Q.DT_BF16, Q.DT_F32, 7, one, 16, one, 16, one, 16, 16, 16, 16, None) == 1
    # scaled: only int8 / fp8 inputs; no int32 output with block scales; reference layout checks divisibility first
    assert lib.qgemm_scaled_gemm(Q.DT_BF16, Q.DT_F32, 1, 0, one, one, one, one, one, 16, 16, 16, 16, 0, None) == 2
    assert lib.qgemm_scaled_gemm(Q.DT_I8, Q.DT_I32, 2, 0, one, one, one, one, one, 16, 16, 16, 16, 0, None) == 2
    assert lib.qgemm_scaled_gemm(Q.DT_F8E4M3, Q.DT_BF16, 2, 1, one, one, one, one, one, 64, 48, 64, 128, 0, None) == 6
    assert lib.qgemm_scaled_gemm(Q.DT_F8E4M3, Q.DT_BF16, 2, 1, one, one, one, one, one, 48, 64, 48, 128, 0, None) == 7
    assert lib.qgemm_scaled_gemm(Q.DT_F8E4M3, Q.DT_BF16, 2, 1, one, one, one, one, one, 64, 64, 64, 80, 0, None) == 8
    assert lib.qgemm_scaled_gemm(Q.DT_F8E4M3, Q.DT_BF16, 2, 0, one, one, one, one, one, 64, 64, 64, 128, -1, None) == 1
    assert lib.qgemm_transpose(3, one, one, 4, 4, None) == 2
    assert lib.qgemm_set_option(b"no_such_option", 1) == 1
    if lib.qgemm_device_count() == 0:
        assert lib.qgemm_init() == 3          # QGEMM_ERR_NO_DEVICE: loud, no CPU fallback
        assert lib.qgemm_gemm(Q.DT_BF16, Q.DT_F32, 1, one, 16, one, 16, one, 16, 16, 16, 16, None) == 3


def test_python_ops_refuse_host_tensors():
    import torch
    a = torch.zeros((16, 16), dtype=torch.int8)
    with pytest.raises(ValueError):
        Q.int8_mm(a, a, torch.ones(1), torch.ones(1), torch.zeros((16, 16), dtype=torch.int32))


@pytest.mark.parametrize("tiles_m,tiles_n", [(32, 32), (1, 1), (1, 9), (7, 5), (24, 18), (3, 100), (48, 36), (2, 7)])
@pytest.mark.parametrize("group", [1, 4, 8, 16])
def test_tile_raster_is_a_bijection(tiles_m, tiles_n, group):
    """XCD remap + GROUP_M raster (replaces sm89_gemm_kernel_v3.cu:169-183): every tile exactly once."""
    total = tiles_m * tiles_n
    seen = {Q.tile_map(w, tiles_m, tiles_n, group) for w in range(total)}
    assert seen == {(i, j) for i in range(tiles_m) for j in range(tiles_n)}
    with pytest.raises(Q.QgemmError):
        Q.tile_map(total, tiles_m, tiles_n, group)


def test_tile_raster_keeps_an_xcd_on_a_compact_cluster():
    """Workgroups w, w+8, w+16, .. share an XCD (and its L2): their first 32 tiles must reuse few A / B panels."""
    tiles_m = tiles_n = 32
    for xcd in range(8):
        first = [Q.tile_map(xcd + 8 * i, tiles_m, tiles_n, 8) for i in range(32)]
        rows = {t[0] for t in first}
        cols = {t[1] for t in first}
        assert len(rows) + len(cols) <= 12      # 8 x 4 cluster: 12 panels for 32 tiles


def test_plan_names_the_kernel_without_a_device():
    """qgemm_plan: the tile / pipeline / K-split choice for the five BASELINE configs and for operands stored
    K-major, from the host (256 CUs assumed).  Pins the heuristic: a change of choice shows up here first."""
    plan = Q.plan
    assert plan(Q.DT_F16, 0, 0, 1024, 1024, 1024) == "skinny_64x64_k8"                       # config 1
    assert plan(Q.DT_F16, 0, 0, 1024, 1024, 512) == "128x32_w4x1_dma"                        # (8 K steps: one per wave)
    assert plan(Q.DT_I8, Q.SCALE_PER_MATRIX, 0, 4096, 4096, 4096) == "256x256_w2x2_solo"     # config 2
    # int8 and 16-bit types: 4 waves when the tiles fill whole rounds of CUs, 8 waves in a partly filled round
    assert plan(Q.DT_I8, Q.SCALE_PER_MATRIX, 0, 3840, 4096, 4096) == "256x256_w2x4_solo8"
    # a partly filled round that 192-row tiles fill better: 3072^3 is 144 tiles of 256 x 256 or 192 of 192 x 256
    assert plan(Q.DT_I8, Q.SCALE_PER_MATRIX, 0, 3072, 3072, 3072) == "192x256_w2x4_solo8"
    assert plan(Q.DT_BF16, 0, 0, 3072, 4096, 4096) == "192x256_w2x4_solo8"
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 1536, 7168, 2048) == "192x256_w2x4_solo8_ks"
    assert plan(Q.DT_BF16, 0, 0, 8192, 4096, 4096) == "256x256_w2x2_solo"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 8192, 8192, 8192) == "256x256_w2x2_solo"  # config 3
    # config 4: the twin of the 8-wave kernel that reads a_scale as this layout passes it (any number of K blocks per row)
    # config 4: 10 column bands on 256 x 256 tiles (240 of them), the 2048 columns to the right on 32 x 8 tiles of 192 x 256
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 6144, 4608, 7168) == "256x256_w2x4_solo8_ks|192x256_w2x4_solo8_ks"
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 6144, 4608, 7168 - 128) == "256x256_w2x4_solo8_ks|192x256_w2x4_solo8_ks"
    # config 5: the skinny-M kernel (K split over the eight waves of a workgroup)
    for m, name in ((16, "skinny_16x32_k8"), (64, "skinny_64x32_k8"), (128, "skinny_64x64_k8")):
        assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, m, 7168, 2048) == name
        assert plan(Q.DT_I8, Q.SCALE_PER_MATRIX, 0, m, 7168, 2048) == name
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 24, 4096, 4096) == "skinny_32x32_k8"
    # ... with a K split across workgroups on top where the strips leave half of the CUs idle and K is long
    assert plan(Q.DT_BF16, 0, 0, 24, 4096, 16384) == "skinny_32x32_k8_splitk2"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 16, 4096, 28672) == "skinny_16x32_k8_splitk2"
    # ... or, up to 32 rows and 32 .. 112 K steps, strips of 16 columns, twice as many and no K split
    assert plan(Q.DT_BF16, 0, 0, 24, 4096, 4096) == "skinny_32x16_k8"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 16, 4096, 14336) == "skinny_16x16_k8"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 16, 2048, 16384) == "skinny_16x32_k8_splitk4"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 64, 2048, 8192) == "skinny_64x32_k8_splitk4"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 16, 8192, 8192) == "skinny_16x32_k8"
    # 33 .. 64 rows whose 32-column strips need a second round of CUs: 64-column strips; 65 .. 128 rows whose strips
    # fit one round and K is not long: the skinny-M kernel rather than what the estimate (of resident operands) likes
    assert plan(Q.DT_BF16, 0, 0, 64, 14336, 4096) == "skinny_64x64_k8"
    assert plan(Q.DT_BF16, 0, 0, 32, 14336, 4096) == "skinny_64x64_k8"          # (from 17 rows on; 16 rows stay on 32-column strips)
    assert plan(Q.DT_BF16, 0, 0, 16, 14336, 4096) == "skinny_16x32_k8"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 64, 8192, 8192) == "skinny_64x32_k8"
    assert plan(Q.DT_BF16, 0, 0, 128, 7168, 2048) == "skinny_64x64_k8"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 128, 8192, 8192) == "skinny_64x64_k8"
    assert plan(Q.DT_BF16, 0, 0, 128, 8192, 8192) == "128x128_w2x2_k2_splitk4"
    # 17 .. 256 rows against few columns, 32 .. 48 K steps: small tiles of the skinny-M kernel over several row tiles, whichever
    # moves least in one round of CUs, instead of a taller tile with a K split (block scales: up to 32 K steps)
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 128, 1024, 4096) == "skinny_32x32_k8"                # (was 128 x 32 with four K slices)
    assert plan(Q.DT_BF16, 0, 0, 128, 2048, 2048) == "skinny_64x32_k8"
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 96, 2048, 4096) == "skinny_32x32_k8"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 130, 1536, 6144) == "skinny_32x32_k8"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 64, 1024, 4096) == "skinny_16x32_k8"                 # (was 64 x 32 with four K slices)
    assert plan(Q.DT_BF16, 0, 0, 48, 2048, 2048) == "skinny_16x32_k8"
    assert plan(Q.DT_BF16, 0, 0, 64, 7168, 2048) == "skinny_64x32_k8"                                    # (wide: one row tile, as before)
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 128, 2048, 7168) == "skinny_128x32_k8_splitk4"       # 56 steps: the split stays
    assert "splitk" in plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 130, 1536, 6144)                            # (block scales: only up to 32 steps)
    Q.set_option("small_tiles", 0)
    try:
        assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 128, 1024, 4096) == "skinny_128x32_k8_splitk4"
    finally:
        Q.set_option("small_tiles", 1)
    # ... but not with few K steps or where the estimate prefers wide tiles
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 128, 7168, 512) == "128x32_w4x1_dma"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 64, 8192, 1024) == "64x32_w4x1_dma"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 16, 1024, 1024) == "skinny_16x32_k8"
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 64, 7168, 2048) == "skinny_64x32_k8"          # block scales too
    assert "skinny" not in plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 128, 28672, 4096)
    # mid sizes: the cost estimate prefers 128 x 128 tiles while they fit in one round of two per CU, and the
    # form with two K groups per workgroup where there are no more tiles than CUs
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 1536, 1536, 1536) == "128x128_w2x2_k2"
    assert plan(Q.DT_I8, Q.SCALE_PER_MATRIX, 0, 2048, 2048, 8192) == "128x128_w2x2_k2"
    assert plan(Q.DT_BF16, 0, 0, 512, 8192, 8192) == "128x128_w2x2_k2"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 2560, 2560, 2560) == "256x128_w2x2_cw"       # 200 tiles: 19.1 us, 128 x 128: 21.0
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 4096, 2048, 2048) == "128x128_w2x2_dma"      # 256 tiles, 16 K steps: 18.1 / 18.8 either way
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 3072, 3072, 3072) == "192x256_w2x4_solo8"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 3840, 4096, 4096) == "256x256_w2x2_solo"
    assert plan(Q.DT_BF16, 0, 0, 512, 4096, 4096) == "64x128_w1x4_k2"
    # one round of 256 x 128 tiles where 256 x 256 tiles would leave half of the CUs idle: the row with copying waves
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 2048, 4096, 4096) == "256x128_w2x2_cw"
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 1024, 8192, 8192) == "256x128_w2x2_cw_ks"
    assert plan(Q.DT_BF16, 0, 0, 1536, 4096, 4096) == "256x128_w2x2_cw"
    # a partly empty last round of 256 x 256 tiles: its rows become a second launch with smaller tiles
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 6400, 6144, 4096) == "256x256_w2x2_solo+256x128_w2x2_cw"
    # (not where smaller tiles make whole rounds by themselves: 6144^3 is 768 tiles of 192 x 256, three rounds, 163.7 us in
    # one launch against 165.9 in two)
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 6144, 6144, 6144) == "192x256_w2x4_solo8"
    # (block scales as this layout passes them: the twin for the first launch, the simple pipeline takes any strides;
    # 6144^3: 210 us in two launches against 229 in one)
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 2560, 7680, 2048) == "256x256_w2x4_solo8_ks+128x128_w2x2_k2"
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 6144, 6144, 6144) == "256x256_w2x4_solo8_ks+256x128_w2x2_cw_ks"
    # ... also when a single launch would take smaller tiles for everything, and with a rest of at most 128 rows
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 5000, 4096, 7168) == "256x256_w2x2_solo+128x128_w2x2_k2"
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 7000, 7168, 2048) == "256x256_w2x2_solo+skinny_64x64_k8"
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 7000, 7168, 2048) == "256x256_w2x4_solo8_ks+skinny_64x64_k8"
    # ... or its columns ("|"), where those divide the full rounds and the rows do not: 16 x 56 tiles are 3.5 rounds, 48
    # column bands exactly three, and the 4096 x 2048 to their right one round of 256 x 128 tiles (176 -> 172 us)
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 4096, 14336, 4096) == "256x256_w2x2_solo|256x128_w2x2_cw"
    assert plan(Q.DT_BF16, 0, 0, 8192, 4608, 4096) == "256x256_w2x2_solo|128x128_w2x2_k2"
    Q.set_option("row_split", 2)            # (2 / 3: the rows / the columns wherever the geometry allows)
    try:
        assert plan(Q.DT_BF16, 0, 0, 8192, 4608, 4096) == "256x256_w2x2_solo+256x128_w2x2_cw"
        Q.set_option("row_split", 3)
        assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 6144, 6144, 6144) == "256x256_w2x2_solo|256x128_w2x2_cw"
    finally:
        Q.set_option("row_split", 1)
    Q.set_option("row_split", 0)
    try:
        assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 6400, 6144, 4096) == "256x256_w2x2_solo"
    finally:
        Q.set_option("row_split", 1)
    # operands stored K-major: read as stored where that is cheaper than transposing, else transposed first
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 3, 2048, 2048, 2048) == "128x128_w2x2_k2_tn"
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 3, 4096, 2048, 2048) == "256x128_w2x2_cw_tn"
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 3, 6144, 4608, 7168) == "transpose+256x256_w2x4_solo8|192x256_w2x4_solo8"
    assert plan(Q.DT_BF16, 0, 2, 1024, 1024, 1024) == "64x128_w1x4_k2_nn"
    assert plan(Q.DT_BF16, 0, 2, 8192, 8192, 8192) == "transpose+256x256_w2x2_solo"
    # large shapes whose transposes are a sizeable part: as stored, on the K-major 256 x 128 row with copying waves
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 3, 4096, 4096, 4096) == "256x128_w2x2_cw_tn"
    assert plan(Q.DT_BF16, 0, 2, 2048, 8192, 8192) == "256x128_w2x2_cw_nn"
    assert plan(Q.DT_I8, Q.SCALE_PER_MATRIX, 2, 1024, 1024, 1024).startswith("transpose+")   # no K-major int8 family
    # K bytes not a multiple of 16: the any-shape kernel; whole 16-byte chunks with a partial last K step: the MFMA kernels
    assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 100, 100, 100) == "strided_any_shape"
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 6144, 4608, 7200) == "256x256_w2x4_solo8_ks|192x256_w2x4_solo8_ks"       # (57 K blocks)
    assert plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 6144, 4608, 7216) == "256x256_w2x4_solo8_ks|192x256_w2x4_solo8_ks"
    assert plan(Q.DT_I8, Q.SCALE_PER_MATRIX, 0, 4096, 4096, 4000) == plan(Q.DT_I8, Q.SCALE_PER_MATRIX, 0, 4096, 4096, 4096)
    assert plan(Q.DT_BF16, 0, 0, 1024, 1024, 1000) == plan(Q.DT_BF16, 0, 0, 1024, 1024, 1024)
    assert plan(Q.DT_BF16, 0, 0, 1024, 1024, 1004) == "strided_any_shape"
    # forced rows are honoured, and a forced split shows in the name
    Q.force_config("128x128_w2x2_dma")
    Q.set_option("force_split", 4)
    try:
        assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 8192, 8192, 8192) == "128x128_w2x2_dma_splitk4"
    finally:
        Q.force_config(None)
        Q.set_option("force_split", 0)
    # a name no family has is refused when it is set; a name the problem's family lacks when a problem asks for it
    with pytest.raises(Q.QgemmError):
        Q.force_config("no_such_row")
    Q.force_config("256x256_w2x2_solo")                          # (not among the block-scaled rows)
    try:
        with pytest.raises(Q.QgemmError):
            plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 6144, 4608, 7168)
        assert plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 6144, 4608, 7168) == "256x256_w2x2_solo"
    finally:
        Q.force_config(None)
    with pytest.raises(Q.QgemmError):
        plan(Q.DT_BF16, Q.SCALE_BLOCK128, 0, 256, 256, 256)      # block scales: fp8 and int8 operands
    with pytest.raises(Q.QgemmError):
        plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 0, 256, 256)


def test_c_abi_header_is_plain_c(tmp_path):
    """include/qgemm.h is the boundary a C, Go (cgo) or Rust (bindgen) caller binds: it has to compile as C99
    with warnings as errors, without any HIP or C++ header."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "use.c"
    src.write_text('#include "qgemm.h"\nint main(void) { char b[8]; return qgemm_plan(0, 0, 0, 1, 1, 1, b, sizeof b) == 12345; }\n')
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(root, "include"),
                    "-c", str(src), "-o", str(tmp_path / "use.o")], check=True)


def test_too_large_is_reported_not_wrapped():
    """Dimensions beyond what the kernels index come back as QGEMM_ERR_TOO_LARGE (9) instead of wrapping around:
    more tiles than a grid holds (plan_nt), a transpose side of 2^31, block scales past 32-bit byte offsets."""
    lib = L.load_library()
    one = C.c_void_p(16)
    with pytest.raises(Q.QgemmError) as e:
        Q.plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 1 << 22, 1 << 22, 128)
    assert e.value.status == 9
    assert lib.qgemm_transpose(2, one, one, 1 << 31, 4, None) == 9
    assert lib.qgemm_transpose(1, one, one, 4, 1 << 31, None) == 9
    # block scales: M * ceil(K / 128) * 4 bytes >= 2^32 cannot go to the MFMA kernel
    assert Q.plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, 1 << 20, 256, 1 << 17) == "strided_any_shape"
    assert b"static scratch" in lib.qgemm_status_string(10)


def test_workspace_entries_need_no_device_to_answer():
    lib = L.load_library()
    base, size = C.c_void_p(123), C.c_size_t(7)
    assert lib.qgemm_workspace_info(C.byref(base), C.byref(size)) == 0
    if lib.qgemm_device_count() == 0:
        assert base.value is None and size.value == 0
        assert lib.qgemm_reserve_workspace(1 << 20) == 3          # QGEMM_ERR_NO_DEVICE
    assert lib.qgemm_workspace_info(None, None) == 1


def test_nt_forwarders_pass_dense_strides_like_the_reference(tmp_path):
    """GEMM_kernel_v3_1 / v4_1 (and the NN entries) ignore the caller's ldA / ldB exactly as the reference's
    launchers do (sm80_gemm_kernel_v3.1.cu:292 passes K for ldB; tests/includes/test_config.h:238 calls every
    entry with ldB = N): built against a stub qgemm_gemm that prints what it receives."""
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    src = tmp_path / "fwd.cpp"
    src.write_text(r'''
#include <cstdio>
#include "gemm.h"
extern "C" int qgemm_gemm(int in_dtype, int out_dtype, int layout_b, const void *, size_t ldA, const void *, size_t ldB,
                          void *, size_t ldC, size_t M, size_t N, size_t K, void *) {
    std::printf("%d %d %d %zu %zu %zu %zu %zu %zu\n", in_dtype, out_dtype, layout_b, ldA, ldB, ldC, M, N, K);
    return 0;
}
extern "C" const char *qgemm_status_string(int) { return ""; }
int main() {
    const __hip_bfloat16 *a = nullptr, *b = nullptr;
    float *c = nullptr;
    GEMM_kernel_v3_1<__hip_bfloat16, float>(a, 64, b, 48, c, 56, 32, 48, 64);   // M=32 N=48 K=64, ldB = N as the harness
    GEMM_kernel_v4_1<__hip_bfloat16, float>(a, 999, b, 999, c, 48, 32, 48, 64);
    GEMM_kernel_v3<__hip_bfloat16, float>(a, 999, b, 999, c, 48, 32, 48, 64);
    return 0;
}
''')
    exe = tmp_path / "fwd"
    subprocess.run([hipcc, "-std=c++17", "--offload-arch=gfx950", "-I", os.path.join(ROOT, "include"), str(src), "-o",
                    str(exe)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split("\n")
    assert out[0] == "1 0 1 64 64 56 32 48 64"      # bf16 -> f32, B is N x K: ldB = K whatever the caller said; ldC kept
    assert out[1] == "1 0 1 64 64 48 32 48 64"
    assert out[2] == "1 0 0 64 48 48 32 48 64"      # B is K x N: ldB = N


def test_fnuz_fp8_is_refused_not_misread():
    """torch.float8_e4m3fnuz (the gfx942 encoding the reference's fp8_mm names) has another bias and another NaN
    code: the wrappers refuse it instead of decoding it as OCP e4m3."""
    import torch
    if not hasattr(torch, "float8_e4m3fnuz"):
        pytest.skip("this torch has no fnuz dtype")
    a = torch.zeros((32, 128), dtype=torch.uint8).view(torch.float8_e4m3fnuz)
    s = torch.ones(1)
    with pytest.raises(TypeError):
        Q.fp8_mm(a, a, s, s, torch.zeros((32, 32), dtype=torch.bfloat16))
    ok = torch.zeros((32, 128), dtype=torch.uint8).view(torch.float8_e4m3fn)
    with pytest.raises(ValueError):          # c with the wrong shape
        Q.fp8_mm(ok, ok, s, s, torch.zeros((32, 16), dtype=torch.bfloat16))
    with pytest.raises(ValueError):          # c with a non-unit inner stride
        Q.fp8_mm(ok, ok, s, s, torch.zeros((32, 64), dtype=torch.bfloat16)[:, ::2])


def test_bench_has_traffic_counters_for_the_headline_kernel():
    """bench.py's roofline.traffic is a constant read off offline counter runs, keyed by kernel name: the kernel the
    planner names for the headline workload has to have an entry (and the file the entry cites has to exist), or the
    bench line would carry a null."""
    import importlib.util
    root = ROOT
    spec = importlib.util.spec_from_file_location("bench_for_test", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    name = Q.plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 8192, 8192, 8192)
    traffic, source = bench.measured_traffic(name, 8192)
    assert traffic and traffic > 2 * 8192 * 8192 + 2 * 8192 * 8192, (name, source)
    cited = [w for w in source.replace(",", " ").split() if w.startswith("profiles/")]
    assert cited and all(os.path.exists(os.path.join(root, f)) for f in cited), source
    assert bench.measured_traffic("no_such_kernel", 8192)[0] is None
