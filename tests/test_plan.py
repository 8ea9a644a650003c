"""Host logic that chooses the launches of a tiled matmul (no GPU needed): one tile shape,
a K split when the caller brings a workspace, or two regions when the last round of the
main shape would leave most of the chip idle."""
import re

from modular_amd import _lib


def parse(text):
    parts = [re.match(r"(\d+)x(\d+) x(\d+)", p.strip()) for p in re.split(r"\+ (?:columns|rows) from \d+:", text)]
    return [(int(m.group(1)), int(m.group(2)), int(m.group(3))) for m in parts]


def test_single_shapes_and_k_split():
    assert _lib.matmul_describe(2048, 6144, 4096) == "256x256 x192 persistent"
    assert _lib.matmul_describe(2040, 6144, 4096) == "256x256 x192"
    assert _lib.matmul_describe(8, 4096, 4096) == "skinny"
    assert _lib.matmul_describe(64, 4096, 4096) == "skinny" and _lib.matmul_describe(32, 28672, 4096) == "skinny"
    # 33 to 64 rows go to the tiles unless the weights are small (under 32 MB): wide matrices, and narrow ones split over K
    assert _lib.matmul_describe(64, 28672, 4096).startswith("128x128")
    assert "K split" in _lib.matmul_describe(48, 8192, 28672) and _lib.matmul_describe(33, 6144, 4096) == "skinny"
    assert _lib.matmul_describe(48, 8192, 28672, True, False) == "skinny"  # no workspace, no split: the streaming kernel
    # 25 to 32 rows: the tiles only where K is long and N narrow
    assert "K split" in _lib.matmul_describe(32, 8192, 28672) and _lib.matmul_describe(24, 8192, 28672) == "skinny"
    assert _lib.matmul_describe(32, 8192, 8192) == "skinny" and _lib.matmul_describe(32, 10240, 16384) == "skinny"
    with_ws, without = _lib.matmul_describe(256, 4096, 14336), _lib.matmul_describe(256, 4096, 14336, True, False)
    assert "K split" in with_ws and "K split" not in without
    # where the pieces of a K split would fill three quarters of the chip with at least 16 slabs each, the four-wave kernel
    # cuts every tile and its blocks exchange their sums inside the one launch
    assert _lib.matmul_describe(256, 7168, 16384) == "128x256 x56 persistent, four waves, every tile cut in pieces of 32 slabs"
    # (not with pieces of 8 slabs, not with eight pieces of 16, not where the rows fill less than three quarters of the tiles)
    assert "K split" in _lib.matmul_describe(1536, 1024, 4096) and "K split" in _lib.matmul_describe(128, 8192, 16384)
    assert "K split" in _lib.matmul_describe(48, 8192, 28672)
    assert _lib.matmul_describe(512, 2048, 28672) == "128x256 x32 persistent, four waves, every tile cut in pieces of 28 slabs"
    assert _lib.lib().maxfp8_matmul_workspace_bytes(256, 7168, 16384) >= 224 * 128 * 256 * 4
    assert _lib.matmul_describe(0, 10, 10) == "nothing to do"


def test_two_regions_cover_the_problem_once(tune):
    tune(MAXFP8_W4="0")  # (the four-wave kernel, which takes such shapes in one launch, has its own test below)
    for (M, N, K) in [(2048, 28672, 4096), (28672, 2048, 4096), (2040, 28600, 4096)]:
        text = _lib.matmul_describe(M, N, K)
        assert " + " in text, text
        cut = int(re.search(r"from (\d+)", text).group(1))
        (bm1, bn1, n1), (bm2, bn2, n2) = parse(text)
        ceil = lambda a, b: -(-a // b)
        if "columns" in text:
            assert cut % bn1 == 0 and 0 < cut < N
            assert n1 == ceil(M, bm1) * (cut // bn1) and n2 == ceil(M, bm2) * ceil(N - cut, bn2)
        else:
            assert cut % bm1 == 0 and 0 < cut < M
            assert n1 == (cut // bm1) * ceil(N, bn1) and n2 == ceil(M - cut, bm2) * ceil(N, bn2)
        assert n1 % 256 == 0, "the first region runs in whole rounds of the 256 CUs"


def test_four_wave_kernel_where_its_tile_count_fits_the_chip(tune):
    # DeepSeek-V3 o_proj at M = 4096: 448 tiles of 256 x 256 are 1.75 rounds of the 256 CUs, 728 tiles of 160 x 256 are 2.84
    assert _lib.matmul_describe(4096, 7168, 16384, True, False) == "160x256 x728 persistent, four waves"
    # with a workspace for the pieces: 616 tiles of 192 x 256 as two whole rounds and 104 tiles in two pieces each
    assert _lib.matmul_describe(4096, 7168, 16384) == "192x256 x616 persistent, four waves, tail cut in pieces of 64 slabs"
    assert _lib.lib().maxfp8_matmul_workspace_bytes(4096, 7168, 16384) >= 256 * 192 * 256 * 4
    # a ragged last column tile is fine as long as C's rows keep their 16-byte alignment (N a multiple of 8): the one matmul
    # over DeepSeek-V3's stacked q_a and kv_a weights, N = 1536 + 576
    assert _lib.matmul_describe(4096, 2112, 7168) == "160x256 x234 persistent, four waves"
    # N not a multiple of 8, an odd number of slabs, and well under one round of tiles stay with the eight-wave shapes
    assert "four waves" not in _lib.matmul_describe(4096, 7164, 16384)
    assert "four waves" not in _lib.matmul_describe(4096, 7168, 16384 + 128)
    assert "four waves" not in _lib.matmul_describe(128, 28672, 4096, False)
    tune(MAXFP8_W4="0")
    assert "four waves" not in _lib.matmul_describe(4096, 7168, 16384)
    tune(MAXFP8_W4="6", MAXFP8_W4_SPLIT="0")
    assert _lib.matmul_describe(4096, 7168, 16384) == "192x256 x616 persistent, four waves"
    # the cut wants a last round of at most half the CUs' number of tiles (216 of 160 x 256 are too many), slabs in fours
    tune(MAXFP8_W4="5", MAXFP8_W4_SPLIT="1")
    assert _lib.matmul_describe(4096, 7168, 16384) == "160x256 x728 persistent, four waves"
    assert "tail cut in pieces of 8 slabs" in _lib.matmul_describe(2040, 6144, 4096)
    assert "tail cut" not in _lib.matmul_describe(2040, 6144, 4096 + 256)
