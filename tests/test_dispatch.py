"""Host-side decisions of the kernel wrappers that need no GPU: which attention kernel takes
a shape, which product kernel takes a row count, what the fault flags say, and the check of
positions against the rotary table."""
import pytest
import torch

from nano_vllm_amd.kernels.library import KernelError
from nano_vllm_amd.kernels.ops import HipKernels, PREFILL_MAX_TABLE, check_positions_fit


def _qo(rows=4, width=256):
    q = torch.zeros((rows, width), dtype=torch.bfloat16)
    return q, width, torch.zeros_like(q), width


def test_prefill_kernel_is_not_chosen_for_block_tables_it_cannot_stage():
    q, qs, out, os_ = _qo()
    takes = HipKernels._prefill_kernel_takes
    assert takes(128, 256, 16, q, qs, out, os_)
    assert takes(128, 8, PREFILL_MAX_TABLE, q, qs, out, os_)
    # pages of 8 tokens and a context of more than 32768: the general kernel runs instead
    assert not takes(128, 8, PREFILL_MAX_TABLE + 1, q, qs, out, os_)
    assert not takes(16, 4, 8, q, qs, out, os_)           # head size 16, pages of 4
    assert not takes(128, 4, 8, q, qs, out, os_)
    assert not takes(128, 256, 8, q, 252, out, os_)       # rows that are not 16-byte aligned


def test_decode_kernel_limits():
    q, qs, out, os_ = _qo()
    takes = HipKernels._decode_kernel_takes
    assert takes(4, 128, 256, q, qs, out, os_) and takes(16, 32, 8, q, qs, out, os_)
    assert not takes(17, 128, 256, q, qs, out, os_)       # more than 16 query heads per kv head
    assert not takes(4, 48, 256, q, qs, out, os_) and not takes(4, 288, 256, q, qs, out, os_)
    assert not takes(4, 128, 12, q, qs, out, os_)


def test_every_fault_flag_has_a_message():
    k = object.__new__(HipKernels)
    for flags, text in ((1, "token id"), (2, "page is missing"), (4, "plan needed more segments"), (8, "unknown flags")):
        k.fault_flag = torch.tensor([flags], dtype=torch.int32)
        with pytest.raises(KernelError, match=text):
            k.check_faults()
        assert int(k.fault_flag) == 0
    k.check_faults()


def test_positions_must_be_rows_of_the_rotary_table():
    table = torch.zeros((128, 16))
    check_positions_fit(table, 16, 128)
    with pytest.raises(KernelError, match="no row in the rotary table of 128"):
        check_positions_fit(table, 16, 129)
    with pytest.raises(KernelError, match="needs max_position"):
        check_positions_fit(table, 16, None)
    check_positions_fit(table, 32, 10)                  # a table narrower than the head: the first 16 channels are rotated
    for head_dim, bad in ((8, table), (16, torch.zeros((128, 7))), (16, torch.zeros((128, 16), dtype=torch.float64))):
        with pytest.raises(KernelError, match="float32"):
            check_positions_fit(bad, head_dim, 10)


def test_row_counts_choose_the_product_kernel():
    k = object.__new__(HipKernels)
    # the thresholds are instance attributes set in __init__, which needs a GPU: the defaults, by hand
    k.own_matmul_rows, k.skinny_max_rows, k.small_weight_bytes = 16, 64, 64 << 20
    k.medium_max_rows, k.medium_max_weight_rows = 224, 8192
    k.team_max_rows, k.team_min_weight_rows, k.product_choice = 16, 8192, {}
    k.tile_for_wide_weights = True
    assert k._own_kernel(1, 4096, 4096) == "skinny" and k._own_kernel(16, 24576, 4096) == "team"
    assert k._own_kernel(16, 24576, 4104) == "skinny"            # k no multiple of 32
    assert k._own_kernel(17, 4096, 4096) == "medium" and k._own_kernel(224, 4096, 12288) == "medium"
    assert k._own_kernel(0, 4096, 4096) is None
    assert k._own_kernel(240, 5120, 25600) is None and k._own_kernel(64, 51200, 5120) == "tile"
    assert k._own_kernel(256, 24576, 4096) == "tile" and k._own_kernel(257, 24576, 4096) is None
    assert k._own_kernel(64, 24576, 4104) is None                # k no multiple of 64
    # what was measured on the model's own weights goes before the rules, per 16 rows, plain and gated apart
    k.product_choice[(5120, 25600, False)] = {15: "medium", 16: "medium", 2: "library"}
    k.product_choice[(51200, 5120, True)] = {4: "skinny"}
    assert k._own_kernel(240, 5120, 25600) == "medium" and k._own_kernel(225, 5120, 25600) == "medium"
    assert k._own_kernel(32, 5120, 25600) is None and k._own_kernel(17, 5120, 25600) is None
    assert k._own_kernel(48, 5120, 25600) == "medium"            # no measurement for 48 rows: the rule
    assert k._own_kernel(64, 51200, 5120, gated=True) == "skinny" and k._own_kernel(64, 51200, 5120) == "tile"
    assert k._own_kernel(8, 5120, 25600) == "skinny"             # up to 16 rows nothing is measured


def test_the_record_of_measured_choices_survives_a_round_trip(tmp_path, monkeypatch):
    from nano_vllm_amd.kernels import ops
    record = tmp_path / "choices.json"
    monkeypatch.setattr(ops, "_choice_file", lambda write=False: str(record) if write or record.exists() else None)
    monkeypatch.setattr(ops, "_product_choices", {})
    assert ops.recorded_product_choices("a GPU") == {}
    ops.recorded_product_choices("a GPU")[(4096, 12288, False)] = {2: "medium", 14: "library"}
    ops.recorded_product_choices("a GPU")[(24576, 4096, True)] = {4: "library"}
    ops._write_product_choices()
    monkeypatch.setattr(ops, "_product_choices", {})
    assert ops.recorded_product_choices("a GPU") == {(4096, 12288, False): {2: "medium", 14: "library"},
                                                     (24576, 4096, True): {4: "library"}}
    assert ops.recorded_product_choices("another GPU") == {}
    record.write_text("not json")
    monkeypatch.setattr(ops, "_product_choices", {})
    assert ops.recorded_product_choices("a GPU") == {}           # an unreadable record: measured again


def test_the_tiled_kernels_workgroups_share_a_weight_out_evenly():
    """Where whole tiles of the LDS-tiled kernel would leave many CUs idle or make a second round that
    few CUs work in, a workgroup takes as many columns as shares the weight out evenly; where most CUs
    have a tile, where a single round has more than 128 rows of x, and where there are many rounds,
    whole tiles stay."""
    from nano_vllm_amd.kernels.ops import HipKernels
    k = HipKernels.__new__(HipKernels)
    k.cus, k.tile_even_shares = 256, True
    assert k._tile_cols(64, 17408, 64, 1) == 40          # 14B gate/up: 272 tiles, two rounds -> 436 workgroups of 40
    assert k._tile_cols(256, 17408, 64, 1) == 40
    assert k._tile_cols(64, 25600, 64, 1) == 56          # 32B gate/up: 400 tiles
    assert k._tile_cols(64, 9728, 64, 1) == 40           # 4B gate/up: 152 tiles, one round
    assert k._tile_cols(256, 9728, 64, 1) == 0           # ... but not with 256 rows of x
    assert k._tile_cols(64, 12288, 64, 1) == 0           # 8B gate/up: 192 of 256 CUs have a tile
    assert k._tile_cols(64, 151936, 128, 1) == 0         # the head: five rounds
    assert k._tile_cols(64, 16384, 64, 1) == 0           # 256 tiles: even as they are
    assert k._tile_cols(64, 17408, 64, 4) == 0           # k cut into ranges: the workgroups are counted otherwise
    k.tile_even_shares = False
    assert k._tile_cols(64, 17408, 64, 1) == 0
