"""The plans of the few-row matrix products are host arithmetic: which kernel, how many blocks
along k.  A plan may depend on the matrix and on the class of the row count (up to 16, 32, 64,
128 rows) only, so that a row's sums come in the same order for every batch of its class; the
consumers of partial sums take at most 8 parts."""
import importlib

import pytest

K = importlib.import_module("daisi-llogos_amd.ops.kernels")

SHAPES = [(24576, 4096), (37888, 3584), (51200, 5120), (59136, 8192),                     # other models' gate/up
          (6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336), (128256, 4096),      # Llama-3.1-8B
          (7168, 5120), (5120, 5120), (34816, 5120), (5120, 17408), (151936, 5120),      # Qwen3-14B
          (10240, 8192), (8192, 8192), (57344, 8192), (8192, 28672),                     # Llama-3.1-70B
          (3072, 2048), (16384, 2048), (2048, 8192), (331, 80), (96, 1000), (17, 8)]


@pytest.mark.parametrize("N,K_", SHAPES)
def test_a_plan_depends_on_the_class_of_the_row_count_only(N, K_):
    for lo, hi in ((1, 4), (5, 8), (9, 16), (17, 32), (33, 64)):
        plans = {K.skinny_plan(M, N, K_) for M in range(lo, hi + 1)}
        if hi <= 16:
            # up to 16 rows the kernel may change with the row count (activations held in
            # registers for the fewest rows), but not within 1..4, 5..8 and 9..16
            assert len(plans) == 1, (N, K_, lo, hi, plans)
        else:
            assert len(plans) == 1 and next(iter(plans))[0] in ("lds", "strips"), (N, K_, lo, hi, plans)
    assert len({K.lds_splits(M, N, K_) for M in range(65, 129)}) == 1


@pytest.mark.parametrize("N,K_", SHAPES)
def test_plans_are_within_what_the_kernels_and_their_consumers_take(N, K_):
    for M in (1, 4, 8, 16, 32, 64, 128):
        parts = K.lds_splits(M, N, K_)
        assert 1 <= parts <= 8
        assert parts == 1 or -(-K_ // 256) >= 2 * parts - 1        # every block along k has work
        if M <= 64:
            kernel, splits, third = K.skinny_plan(M, N, K_)
            assert kernel in ("stationary", "regs", "lds", "strips") and 1 <= splits <= 8 and third >= 1
            if kernel == "strips":
                blocks = -(-(-(-N // 16)) // third) * splits
                assert 16 < M and 5 <= third <= 9 and K_ % 64 == 0 and 0.75 * 512 <= blocks <= 512
            if kernel == "stationary":
                assert M <= 16 and K_ <= 8192 and 2 <= third <= 16
    assert 2 <= K.stationary_strips(N, K_) <= 16


def test_known_choices():
    """The choices measured to be best at the Llama-3.1-8B layer sizes (they are what the
    scoring was fitted to; a change of the scoring that moves them should be a decision)."""
    assert K.skinny_plan(8, 28672, 4096)[0] == "stationary"
    assert K.skinny_plan(8, 4096, 14336) == ("lds", 8, 1)
    assert K.skinny_plan(8, 4096, 4096) == ("lds", 8, 1)
    assert K.skinny_plan(64, 28672, 4096) == ("lds", 1, 1)
    assert K.skinny_plan(64, 6144, 4096) == ("lds", 4, 1)
    assert K.lds_splits(128, 4096, 14336) == 8
    # tall matrices whose blocks of 5 to 9 strips are all resident at once: operands straight into LDS
    assert K.skinny_plan(32, 34816, 5120) == ("strips", 2, 9) and K.skinny_plan(64, 34816, 5120) == ("strips", 2, 9)
    assert K.skinny_plan(64, 57344, 8192) == ("strips", 1, 7)
    assert K.skinny_plan(16, 57344, 8192)[0] == "stationary" and K.skinny_plan(64, 128256, 4096)[0] == "lds"
    assert K.skinny_plan(64, 24576, 4096) == ("strips", 2, 6) and K.skinny_plan(32, 37888, 3584) == ("strips", 1, 5)
    assert K.skinny_plan(64, 51200, 5120) == ("strips", 1, 7) and K.skinny_plan(64, 59136, 8192) == ("strips", 1, 8)
    # ... and not where the LDS few-row product's own blocks fill one round well, or the matrix is small
    assert K.skinny_plan(64, 28672, 4096)[0] == "lds" and K.skinny_plan(32, 28672, 4096)[0] == "lds"
    assert K.skinny_plan(64, 16384, 3072)[0] == "lds" and K.skinny_plan(64, 19456, 2560)[0] == "lds"


def test_sets_of_waves_of_the_prompt_attention():
    """Two sets of waves a block where one prompt's last tile would set the time, one where the
    work of all tiles does (the measured cases at 32 heads)."""
    for lens, want in (([512], 2), ([1536], 2), ([2048], 2), ([2560], 1), ([4096], 1), ([16384], 1),
                       ([1024] * 2, 2), ([512] * 4, 1), ([256] * 4, 2), ([512] * 8, 1)):
        assert K.prefill_halves(lens, None, 32) == want, lens
    # a continued prompt counts the pages before it
    assert K.prefill_halves([128], [4000], 32) == 2 and K.prefill_halves([128] * 64, [4000] * 64, 32) == 1


def test_where_the_tiled_product_serves_prompts(monkeypatch):
    """By default the tiled product takes the gate/up product with its SwiGLU epilogue at 1,024 to 2,048 rows and
    k up to 5,120, and plain products only for matrices much longer than high at 129 to 1,024 rows, in parts of
    k that hold at least two stages of 64."""
    assert K.PROMPT_PRODUCT == "auto"
    assert K.tiles_serve_gated(1024, 4096) and K.tiles_serve_gated(2048, 5120) and not K.tiles_serve_gated(1023, 4096)
    assert not K.tiles_serve_gated(2049, 4096) and not K.tiles_serve_gated(2048, 8192)
    down = (4096, 14336)
    assert K.tiles_plan(64, *down) is None and K.tiles_plan(128, *down) is None          # the few-row products' rows
    assert K.tiles_plan(129, *down) == (4, 2) and K.tiles_plan(256, *down) == (4, 2)
    assert K.tiles_plan(300, *down) == (4, 0) and K.tiles_plan(1024, *down) == (2, 0)
    assert K.tiles_plan(1025, *down) is None
    assert K.tiles_plan(300, 4096, 4096) is None and K.tiles_plan(300, 6144, 4096) is None   # o, qkv: the library's
    assert K.tiles_plan(300, 64, 320) == (2, 0)                                          # 5 stages of 64: not 4 parts
    assert K.tiles_plan(300, 64, 200) is None                                            # k no multiple of 64
    monkeypatch.setattr(K, "PROMPT_PRODUCT", "library")
    assert K.tiles_plan(300, *down) is None and not K.tiles_serve_gated(4096)
    monkeypatch.setattr(K, "PROMPT_PRODUCT", "tiles")
    assert K.tiles_plan(300, 4096, 4096) == (1, 0) and K.tiles_serve_gated(65)


def test_where_the_product_that_adds_itself_to_the_stream_serves():
    """The one-pass product whose blocks own 16 or 32 rows of w and all of k serves up to 16 rows where its
    blocks fill the compute units evenly (256 of them here): one strip a block up to 256 strips (1B, 3B, 8B), two
    above (14B, 70B); the 14B down projection (160 blocks, 89 M weights) only up to 4 rows; never more than 16
    rows or a k that is no multiple of 8; tiny matrices always."""
    plan = lambda M, N, K_: K.residual_plan(M, N, K_, n_cus=256)
    for M in (1, 8, 16):
        assert plan(M, 4096, 4096) == (8, 1) and plan(M, 4096, 14336) == (8, 1)         # 8B
        assert plan(M, 2048, 2048) == (8, 1) and plan(M, 2048, 8192) == (8, 1)          # 1B
        assert plan(M, 3072, 3072) == (8, 1) and plan(M, 3072, 8192) == (8, 1)          # 3B
        assert plan(M, 8192, 8192) == (8, 2) and plan(M, 8192, 28672) == (8, 2)         # 70B
        assert plan(M, 5120, 5120) == (8, 2)                                             # 14B o
        assert plan(M, 5120, 17408) == ((8, 2) if M <= 4 else (0, 0))                    # 14B down
        assert plan(M, 1024, 8192) == (0, 0)                                             # 64 blocks on 256 units
        assert plan(M, 120, 384) == (4, 1) and plan(M, 64, 176) == (4, 1)               # tiny: only the kernel count matters
        assert plan(M, 4096, 4100) == (0, 0)
    assert plan(17, 4096, 4096) == (0, 0) and plan(0, 4096, 4096) == (0, 0)
    assert K.residual_plan(8, 4096, 4096, n_cus=64) == (8, 2)                            # fewer units: two strips a block
