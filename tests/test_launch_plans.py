"""Launch arithmetic checked on the CPU: the grid a launcher asks for must be exactly what its kernel's decode of the
workgroup index assumes.  libsthip.so computes both with the same functions the GPU path uses (no device is touched)."""
import itertools

import pytest

from spiraltorch_amd import hip


def test_row_blocks_of_a_large_lhs_are_never_empty():
    # An A of 2 GiB or more is cut into row blocks of at least 256 rows whose bytes stay below 2^31; where 256 rows
    # do not fit, the answer is 0 and the product keeps the 64-bit-addressed kernels (a block of 0 rows once made the
    # host loop forever: f32 k = 2088961..2097151, bf16 k = 4177921..4194303).
    for elem in (4, 2):
        limit = (1 << 31) // (256 * elem)
        ks = list(range(1, 64)) + [511, 512, 4096, 50257, 1 << 20, limit - 8192, limit - 1, limit, limit + 1,
                                   2 * limit, (1 << 31) // elem, (1 << 31) // elem + 1]
        ks += list(range(limit - 8200, limit + 3, 97))
        for k in ks:
            block = hip.gemm_row_block(k, elem)
            if 256 * k * elem < (1 << 31):
                assert block >= 256 and block % 256 == 0, (k, elem, block)
                assert block * k * elem < (1 << 31)
                assert (block + 256) * k * elem >= (1 << 31)  # the largest such block
            else:
                assert block == 0, (k, elem, block)
    assert hip.gemm_row_block(2090000, 4) == 256  # the shape of the report: 300 x 128 x 2090000
    assert hip.gemm_row_block(0, 4) == 0


CONTEXTS = (1, 2, 3, 7, 8, 12, 16, 64, 128, 256, 257)
SEQUENCES = (1, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300, 511, 512, 1000, 1024, 2048, 2049, 4096)


@pytest.mark.parametrize("causal,biased", [(False, False), (True, False), (False, True), (True, True)])
def test_attention_grid_decodes_to_every_item_once_and_to_nothing_else(causal, biased):
    for contexts, seq, dim in itertools.product(CONTEXTS, SEQUENCES, (32, 64, 128)):
        plan = hip.attention_f32_launch_plan(contexts, seq, dim, causal, biased)
        where = (contexts, seq, dim, causal, biased, plan)
        assert plan["kernel"] in ("general", "fast", "fast_biased", "tiny"), where
        assert plan["consistent"] == 1, where
        assert plan["out_of_range"] == 0 and plan["duplicates"] == 0, where
        assert plan["items"] == plan["items_expected"], where
        if plan["key_splits"] > 1:
            assert plan["keys_per_split"] % 64 == 0 and plan["keys_per_split"] >= 128, where


def test_the_shape_that_once_read_past_its_operands_keeps_the_pairing():
    # 256 contexts of 256 keys, causal: a split would give every tile one chunk, so the launch keeps tile pairs
    plan = hip.attention_f32_launch_plan(256, 256, 64, True, False)
    assert plan["kernel"] == "fast" and plan["key_splits"] == 1 and plan["workgroups"] == 256
    assert plan["out_of_range"] == 0 and plan["items"] == plan["items_expected"] == 512
    # few contexts, long sequence: (tile, chunk) items
    plan = hip.attention_f32_launch_plan(8, 2048, 128, True, False)
    assert plan["key_splits"] > 1 and plan["items"] == plan["items_expected"] == plan["workgroups"]
    # the reference's caller: one context with a bias matrix, keys split over workgroups
    plan = hip.attention_f32_launch_plan(1, 2048, 64, False, True)
    assert plan["kernel"] == "fast_biased" and plan["key_splits"] > 1 and plan["workgroups"] == 16 * plan["key_splits"]


def test_bf16_tile_grids_decode_to_every_split_and_tile_once():
    # few tiles under a long k are split over workgroups: every (k-split, tile) the grid decodes to must exist, have
    # k-tiles to walk, and be decoded exactly once — also where the XCD remap reorders the workgroups
    ms = (1, 33, 64, 65, 100, 255, 256, 257, 300, 512, 1000, 1024, 2048, 4096, 16384)
    ns = (128, 256, 384, 512, 1000, 1536, 2048, 4096, 50257)
    ks = (64, 128, 512, 576, 1024, 2048, 4096, 8192, 65536)
    for m, n, k in itertools.product(ms, ns, ks):
        plan = hip.gemm_bf16_tile_plan(m, n, k)
        where = (m, n, k, plan)
        assert plan["consistent"] == 1, where
        assert plan["out_of_range"] == 0 and plan["duplicates"] == 0, where
        assert plan["items"] == plan["workgroups"] == plan["tiles_m"] * plan["tiles_n"] * plan["k_splits"], where
        assert plan["k_splits"] * plan["k_tiles_per_split"] >= k // 64 > (plan["k_splits"] - 1) * plan["k_tiles_per_split"], where
    assert hip.gemm_bf16_tile_plan(100, 4096, 4096)["k_splits"] > 1       # a batch of 100 rows against a large weight
    assert hip.gemm_bf16_tile_plan(4096, 4096, 4096)["k_splits"] == 1     # BASELINE config 4: 256 tiles of 256×256
    with pytest.raises(hip.HipErr):
        hip.gemm_bf16_tile_plan(128, 128, 100)                            # k not a multiple of 64: another kernel family
