"""Each HIP kernel alone against its plain torch version (tests/torch_kernels.py), in
float32 and bfloat16, at sizes other than the engine's tiny models: widths and vocabularies
that are no power of two, head sizes in steps of 16, odd numbers of heads and groups, page
sizes from 4 to 256, rows that are not aligned for vector access."""
import math
import random
from types import SimpleNamespace

import pytest
import torch

import plain_qwen3 as plain
from nano_vllm_amd.kernels.ops import v_cache_shape
from torch_kernels import TorchKernels, new_caches

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
DEV = "cuda:0"


@pytest.fixture(scope="module")
def hip():
    from nano_vllm_amd.kernels import HipKernels
    return {dt: HipKernels(DEV, dt, quiet=True) for dt in DTYPES}


@pytest.fixture(scope="module")
def ref():
    return TorchKernels(DEV)


def _close(got, want, dtype, what=""):
    got, want = got.float(), want.float()
    scale = float(want.abs().max()) or 1.0
    tol = 2e-6 if dtype == torch.float32 else 2.0 ** -7          # two units in the last place of bfloat16
    err = float((got - want).abs().max()) / scale
    assert err <= tol, f"{what}: error {err:.3e} of the largest value exceeds {tol:.1e}"


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (scale * torch.randn(shape, generator=g)).to(dtype).to(DEV)


# ------------------------------------------------------------------------------ rows
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width,n", [(50, 100, 7), (1000, 4096, 33), (17, 6, 5), (300, 1001, 64)])
def test_embedding(hip, ref, dtype, rows, width, n):
    table = _rand((rows, width), dtype, 1)
    ids = torch.randint(0, rows, (n,), dtype=torch.int32, device=DEV)
    assert torch.equal(hip[dtype].embedding(table, ids), ref.embedding(table, ids))
    # a strided view of a wider tensor (rows not aligned for vector access)
    wide = _rand((rows, width + 3), dtype, 2)
    assert torch.equal(hip[dtype].embedding(wide[:, 1:width + 1], ids), wide[:, 1:width + 1][ids.long()])


def test_embedding_flags_an_id_outside_the_table(hip):
    from nano_vllm_amd.kernels import KernelError
    k = hip[torch.float32]
    table = _rand((10, 8), torch.float32, 1)
    out = k.embedding(table, torch.tensor([3, 10, -1], dtype=torch.int32, device=DEV))
    assert torch.equal(out[0], table[3]) and float(out[1:].abs().max()) == 0.0
    with pytest.raises(KernelError, match="vocabulary"):
        k.check_faults()
    k.check_faults()                                              # the flag is cleared


# ------------------------------------------------------------------------------ norms
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width", [(1, 7), (5, 96), (33, 120), (3, 4096), (2, 5120), (4, 1001)])
@pytest.mark.parametrize("weight32", [False, True])
def test_rms_norm_and_fused_add(hip, ref, dtype, rows, width, weight32):
    x, r = _rand((rows, width), dtype, 3, 2.0), _rand((rows, width), dtype, 4, 3.0)
    w = (1 + 0.1 * torch.randn(width)).to(torch.float32 if weight32 else dtype).to(DEV)
    _close(hip[dtype].rms_norm(x, w, 1e-5), ref.rms_norm(x, w, 1e-5), dtype, "rms_norm")
    r1, r2 = r.clone(), r.clone()
    y1, _ = hip[dtype].add_rms_norm(x, r1, w, 1e-6)
    y2, _ = ref.add_rms_norm(x, r2, w, 1e-6)
    _close(y1, y2, dtype, "add_rms_norm")
    _close(r1, r2, dtype, "residual")
    # in place on the input, as the block calls it
    x2 = x.clone()
    y3, _ = hip[dtype].add_rms_norm(x2, r.clone(), w, 1e-6, out=x2)
    assert torch.equal(y3, y1)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rms_norm_on_strided_rows(hip, ref, dtype):
    big = _rand((6, 300), dtype, 5)
    x = big[:, 3:203]                                              # unaligned start, stride 300
    w = _rand((200,), dtype, 6)
    _close(hip[dtype].rms_norm(x, w, 1e-6), ref.rms_norm(x, w, 1e-6), dtype)


# ------------------------------------------------------------------------------ feed-forward
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,inner", [(1, 5), (7, 160), (3, 12288), (40, 1000)])
def test_silu_mul(hip, ref, dtype, rows, inner):
    x = _rand((rows, 2 * inner), dtype, 7, 2.0)
    _close(hip[dtype].silu_mul(x), ref.silu_mul(x), dtype)


@pytest.mark.parametrize("m,n,k", [(1, 7, 5), (3, 130, 67), (65, 64, 128), (200, 300, 1000), (2, 1001, 96), (64, 96, 4096)])
def test_linear_float32(hip, ref, m, n, k):
    x, w = _rand((m, k), torch.float32, 8), _rand((n, k), torch.float32, 9)
    want = x.double() @ w.double().T
    # a float sum of k terms: each output may be off by about sqrt(k) roundings of its |terms|
    bound = (x.double().abs() @ w.double().abs().T) * (math.sqrt(k) * 2.0 ** -23) + 1e-30
    got = hip[torch.float32].linear(x, w).double()
    assert bool(((got - want).abs() <= bound).all()), float(((got - want).abs() / bound).max())
    b = _rand((n,), torch.float32, 10)
    got = hip[torch.float32].linear(x, w, b).double()
    assert bool(((got - want - b.double()).abs() <= bound + b.double().abs() * 2.0 ** -23).all())


def test_linear_float32_does_not_depend_on_the_rows_beside_it(hip):
    x, w = _rand((70, 333), torch.float32, 11), _rand((129, 333), torch.float32, 12)
    k = hip[torch.float32]
    whole = k.linear(x, w)
    assert torch.equal(k.linear(x[17:18], w), whole[17:18])         # bit for bit: the order of the sum is fixed
    assert torch.equal(k.linear(x[:3], w), whole[:3])
    # every tile shape of the kernel: many rows on a wide weight (128 x 128), fewer (64 x 64), up to 16
    # rows on a weight of few rows (16 x 16) and on one of many (16 x 64)
    x, w = _rand((2100, 77), torch.float32, 13), _rand((17000, 77), torch.float32, 14)
    whole = k.linear(x, w)
    want = x.double() @ w.double().T
    assert float((whole.double() - want).abs().max()) <= 1e-5 * float(want.abs().max())
    assert torch.equal(k.linear(x[1999:2049], w), whole[1999:2049])
    assert torch.equal(k.linear(x[5:6], w), whole[5:6])
    assert torch.equal(k.linear(x[40:56], w[:1000]), whole[40:56, :1000])
    assert torch.equal(k.linear(x[:100], w[300:500]), whole[:100, 300:500])


@pytest.mark.parametrize("m,n,k", [(1, 1001, 96), (5, 384, 120), (70, 777, 256), (3, 64, 4096)])
def test_linear_bfloat16_with_float_result(hip, m, n, k):
    x, w = _rand((m, k), torch.bfloat16, 13), _rand((n, k), torch.bfloat16, 14)
    got = hip[torch.bfloat16].linear(x, w, out_float32=True)
    assert got.dtype == torch.float32
    bound = (x.double().abs() @ w.double().abs().T) * (math.sqrt(k) * 2.0 ** -23) + 1e-30
    assert bool(((got.double() - x.double() @ w.double().T).abs() <= bound).all())


@pytest.mark.parametrize("m,n,k", [(1, 130, 67), (8, 96, 200), (300, 257, 120)])
def test_linear_bfloat16(hip, ref, m, n, k):
    x, w = _rand((m, k), torch.bfloat16, 15), _rand((n, k), torch.bfloat16, 16)
    _close(hip[torch.bfloat16].linear(x, w), ref.linear(x, w), torch.bfloat16)


@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (8, 6144, 4096), (64, 320, 12288), (17, 1000, 264), (33, 24, 8),
                                   (5, 130, 72), (48, 40000, 1288), (20, 40004, 2304), (64, 4096, 4096),
                                   (2, 1000, 1288), (4, 40004, 2304), (3, 130, 72), (4, 4096, 12288),
                                   (100, 1000, 264), (128, 4096, 4096), (120, 130, 72), (90, 4100, 1288), (40, 8192, 512),
                                   (129, 1000, 264), (200, 4096, 4096), (224, 130, 1288), (161, 72, 8)])
def test_linear_bfloat16_few_rows_streams_the_weights(hip, ref, m, n, k):
    """The decode-step product (few rows, k split over workgroups) against a double product."""
    x, w = _rand((m, k), torch.bfloat16, 21), _rand((n, k), torch.bfloat16, 22, 0.05)
    want = x.double() @ w.double().T
    bound = (x.double().abs() @ w.double().abs().T) * (math.sqrt(k) * 2.0 ** -23) + 1e-30
    got32 = hip[torch.bfloat16].linear(x, w, out_float32=True)
    assert bool(((got32.double() - want).abs() <= bound).all())
    got = hip[torch.bfloat16].linear(x, w)
    assert got.dtype == torch.bfloat16
    _close(got, want.float().to(torch.bfloat16), torch.bfloat16)
    b = _rand((n,), torch.bfloat16, 23)
    _close(hip[torch.bfloat16].linear(x, w, b), (want + b.double()).float().to(torch.bfloat16), torch.bfloat16)


@pytest.mark.parametrize("m", [1, 8, 17, 64])
def test_logits_of_a_vocabulary_of_151936(hip, m):
    """The output head at its real size (151936 x 4096, float result): one row and eight through
    the weight-streaming kernel, 17 and 64 through the path for many wanted places, each against
    a double product, and the argmax of every row with it."""
    n, k = 151936, 4096
    x = _rand((m, k), torch.bfloat16, 51)
    gen = torch.Generator(device=DEV).manual_seed(52)
    w = torch.empty((n, k), dtype=torch.bfloat16, device=DEV).normal_(0, 0.02, generator=gen)
    got = hip[torch.bfloat16].linear(x, w, out_float32=True)
    assert got.dtype == torch.float32 and got.shape == (m, n)
    want = torch.empty((m, n), dtype=torch.float64, device=DEV)
    bound = torch.empty((m, n), dtype=torch.float64, device=DEV)
    xd = x.double()
    for lo in range(0, n, 16384):                      # in slices: the weight in double would not be small
        wd = w[lo:lo + 16384].double()
        want[:, lo:lo + 16384] = xd @ wd.T
        bound[:, lo:lo + 16384] = (xd.abs() @ wd.abs().T) * (math.sqrt(k) * 2.0 ** -23)
    # every column was written, the last ones too, each within a float sum's rounding
    assert bool(((got.double() - want).abs() <= bound).all()), float(((got.double() - want).abs() / bound).max())
    assert torch.equal(got.argmax(-1), want.argmax(-1))
    hip[torch.bfloat16].check_faults()


@pytest.mark.parametrize("m,inner,k", [(1, 12288, 4096), (8, 200, 96), (64, 160, 256), (100, 64, 128), (5, 8196, 264),
                                       (40, 9004, 1288), (16, 12288, 4096), (2, 8196, 264), (4, 9004, 1288), (3, 200, 96),
                                       (24, 12288, 4096), (32, 8196, 264), (17, 200, 96)])
def test_linear_silu_mul(hip, ref, m, inner, k):
    x, w = _rand((m, k), torch.bfloat16, 24), _rand((2 * inner, k), torch.bfloat16, 25, 0.1)
    _close(hip[torch.bfloat16].linear_silu_mul(x, w), ref.linear_silu_mul(x, w), torch.bfloat16)
    xf, wf = x.float(), w.float()
    _close(hip[torch.float32].linear_silu_mul(xf, wf), ref.linear_silu_mul(xf, wf), torch.float32)


@pytest.mark.parametrize("teams", [256, 3])
@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (3, 200, 96), (8, 6144, 4096), (16, 4096, 12288), (5, 1000, 5120),
                                   (7, 264, 160), (2, 304, 1632), (4, 1000, 25600), (16, 1016, 6144), (9, 2000, 8192),
                                   (1, 24576, 4096), (11, 72, 17408)])
def test_the_kernel_for_wide_weights_and_few_rows_in_every_form(m, n, k, teams):
    """The kernel whose waves split k inside a workgroup, forced for every weight: x kept in
    registers (several blocks of weight rows a workgroup) and loaded beside the weight (one
    block, or k beyond the registers), one pass and several over a wave's slice of k, slices
    that do not divide, more blocks than lie in LDS at once (3 workgroups), element and float
    results, bias, the SwiGLU gating, strided rows of x; each against a double product."""
    from nano_vllm_amd.kernels import HipKernels
    kern = HipKernels(DEV, torch.bfloat16, quiet=True)
    kern.team_min_weight_rows, kern.teams = 0, teams
    assert kern._own_kernel(m, n, k) == "team"
    wide = _rand((m, k + 8), torch.bfloat16, 61)
    x = wide[:, 8:]                                       # rows 16 bytes off the allocation's start
    w, b = _rand((n, k), torch.bfloat16, 62, 0.05), _rand((n,), torch.bfloat16, 63)
    want = x.double() @ w.double().T
    bound = (x.double().abs() @ w.double().abs().T) * (math.sqrt(k) * 2.0 ** -23) + 1e-30
    got32 = kern.linear(x, w, out_float32=True)
    assert bool(((got32.double() - want).abs() <= bound).all())
    _close(kern.linear(x, w), want.float().to(torch.bfloat16), torch.bfloat16)
    _close(kern.linear(x, w, b), (want + b.double()).float().to(torch.bfloat16), torch.bfloat16)
    gu = want.float().to(torch.bfloat16).float()          # the projection is rounded before the gating
    gated = torch.nn.functional.silu(gu[:, :n // 2]) * gu[:, n // 2:]
    _close(kern.linear_silu_mul(x, w), gated, torch.bfloat16)
    # rows beyond m never reach the result: the same rows beside others
    if m < 16:
        more = torch.cat([x, _rand((16 - m, k), torch.bfloat16, 64, 30.0)])
        assert torch.equal(kern.linear(more, w, out_float32=True)[:m], got32)
    kern.check_faults()


def test_the_product_kernel_is_chosen_by_measurement_and_every_choice_is_right():
    """choose_products times the library against the engine's kernel on the given weights and fills
    a table per (shape, gated) and 16 rows; whatever it chose, and each choice forced, gives the
    product of a double computation, plain and gated."""
    from nano_vllm_amd.kernels import HipKernels
    kern = HipKernels(DEV, torch.bfloat16, quiet=True)
    n, k = 4096, 1024
    weights = [_rand((n, k), torch.bfloat16, 70 + i, 0.05) for i in range(3)]
    small = _rand((64, 64), torch.bfloat16, 75)                     # below min_elements: not measured
    kern.product_choice = {}                                        # a table of its own, and no record of it
    table = kern.choose_products(weights + [small, weights[0].float()], max_rows=80, record=False)
    assert set(table) == {(n, k, False), (n, k, True)}
    for gated in (False, True):
        assert set(table[(n, k, gated)]) == {2, 3, 4, 5} and set(table[(n, k, gated)].values()) <= {"library", "medium", "tile"}
    x = _rand((40, k), torch.bfloat16, 76)
    want = x.double() @ weights[1].double().T
    gu = want.float().to(torch.bfloat16).float()
    gated_want = torch.nn.functional.silu(gu[:, :n // 2]) * gu[:, n // 2:]
    for forced in (None, "library", "medium", "tile"):
        if forced:
            kern.product_choice = {(n, k, g): {b: forced for b in range(2, 6)} for g in (False, True)}
            assert kern._own_kernel(40, n, k) == (None if forced == "library" else forced)
        _close(kern.linear(x, weights[1]), want.float().to(torch.bfloat16), torch.bfloat16, str(forced))
        _close(kern.linear_silu_mul(x, weights[1]), gated_want, torch.bfloat16, str(forced))
        got = kern.linear(x, weights[1], deferred=True)
        _close(got.tensor() if hasattr(got, "tensor") else got, want.float().to(torch.bfloat16), torch.bfloat16, str(forced))
    kern.check_faults()


def test_the_measured_choice_is_kept_with_a_margin_and_recorded(tmp_path, monkeypatch):
    """The rule's kernel stays unless the other one is faster by more than the margin; what was
    chosen is written beside the compiled libraries and read by the next process (here: after the
    process's table is emptied), which measures nothing again."""
    import json
    from nano_vllm_amd.kernels import HipKernels, ops
    record = tmp_path / "product_choice.json"
    monkeypatch.setattr(ops, "_choice_file", lambda write=False: str(record) if write or record.exists() else None)
    monkeypatch.setattr(ops, "_product_choices", {})
    kern = HipKernels(DEV, torch.bfloat16, quiet=True)
    assert kern.product_choice == {}
    n, k = 2048, 2048
    weights = [_rand((n, k), torch.bfloat16, 80 + i, 0.05) for i in range(3)]
    kern.choice_margin = 1.0                   # nothing is faster by 100 %: the rule's kernel (few weight rows: "medium") stays
    table = kern.choose_products(weights, max_rows=48)
    assert table[(n, k, False)] == {2: "medium", 3: "medium"} and table[(n, k, True)] == {2: "medium", 3: "medium"}
    name = torch.cuda.get_device_properties(0).name
    assert json.loads(record.read_text())[name][f"{n},{k},0"] == {"2": "medium", "3": "medium"}
    # the next process: its table comes from the record, and rows it holds are not measured again
    monkeypatch.setattr(ops, "_product_choices", {})
    again = HipKernels(DEV, torch.bfloat16, quiet=True)
    assert again.product_choice[(n, k, True)] == {2: "medium", 3: "medium"}
    again.choice_margin = -1e9                 # a measurement now keeps the fastest, whatever the rule says
    table = again.choose_products(weights, max_rows=64)
    assert table[(n, k, False)][2] == "medium" and table[(n, k, False)][3] == "medium"
    assert table[(n, k, False)][4] in ("library", "medium", "tile")
    assert json.loads(record.read_text())[name][f"{n},{k},0"]["4"] == table[(n, k, False)][4]
    assert HipKernels(DEV, torch.bfloat16, quiet=True).product_choice is again.product_choice     # one table per process


def test_the_kernel_for_wide_weights_refuses_what_it_does_not_take():
    from nano_vllm_amd.kernels import HipKernels
    kern = HipKernels(DEV, torch.bfloat16, quiet=True)
    kern.team_min_weight_rows = 0
    assert kern._own_kernel(17, 9000, 4096) != "team" and kern._own_kernel(4, 9000, 4104) != "team"
    x, w = _rand((4, 4104), torch.bfloat16, 65), _rand((9000, 4104), torch.bfloat16, 66, 0.05)
    _close(kern.linear(x, w), (x.double() @ w.double().T).float().to(torch.bfloat16), torch.bfloat16)


@pytest.mark.parametrize("waves,row_tiles", [(4, 1), (4, 2), (4, 3), (3, 1), (3, 2), (3, 3)])
@pytest.mark.parametrize("m,n,k,splits", [(128, 512, 1024, 1), (70, 200, 264, 2), (17, 4096, 4096, 8), (97, 72, 8, 1),
                                          (256, 512, 1024, 2), (150, 200, 264, 1), (241, 136, 4096, 4), (33, 1000, 520, 1),
                                          (96, 328, 1288, 3), (48, 24, 96, 1)])
def test_the_kernel_for_medium_row_counts_in_every_form(hip, m, n, k, splits, waves, row_tiles):
    """Unsplit and split over k, three and four waves of one to three blocks of weight rows each
    (where the kernel is built with them: up to 96 rows of x all, up to 224 rows four waves of one or
    two blocks, beyond that of one), plain and gated."""
    kern = hip[torch.bfloat16]
    blocks_of_x = ((m + 15) // 16 + 1) // 2 * 2
    if (blocks_of_x > 6 and (waves == 3 or row_tiles == 3)) or (blocks_of_x > 14 and row_tiles == 2):
        from nano_vllm_amd.kernels import KernelError
        kern.medium_shape = (waves, row_tiles, 1)
        try:
            with pytest.raises(KernelError, match="not built"):
                kern._linear_medium(_rand((m, k), torch.bfloat16, 41), k, _rand((n, k), torch.bfloat16, 42), k, None,
                                    torch.empty((m, n), dtype=torch.bfloat16, device=DEV), n, False, False, m, n, k)
        finally:
            kern.medium_shape = None
        return
    x, w = _rand((m, k), torch.bfloat16, 41), _rand((n, k), torch.bfloat16, 42, 0.05)
    want = x.double() @ w.double().T
    kern.medium_shape = (waves, row_tiles, splits)
    try:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
        kern._linear_medium(x, k, w, k, None, out, n, False, False, m, n, k)
        _close(out, want.float().to(torch.bfloat16), torch.bfloat16)
        gated = torch.empty((m, n // 2), dtype=torch.bfloat16, device=DEV)
        kern._linear_medium(x, k, w, k, None, gated, n // 2, False, True, m, n, k)
        y = want.float().to(torch.bfloat16).float()
        _close(gated, (torch.nn.functional.silu(y[:, :n // 2]) * y[:, n // 2:]).to(torch.bfloat16), torch.bfloat16)
        got = kern._linear_medium(x, k, w, k, None, None, 0, False, False, m, n, k, defer=True)
        _close(got.tensor() if hasattr(got, "tensor") else got, want.float().to(torch.bfloat16), torch.bfloat16)
    finally:
        kern.medium_shape = None
    kern.check_faults()


# tile shapes of nva_linear_tile: (rows of x, rows of W, fed by a fifth wave, places of its x ring)
TILE_SHAPES = {0: (64, 128, True, 3), 1: (64, 128, True, 3), 2: (128, 128, True, 3), 3: (256, 128, True, 3),
               4: (64, 256, True, 3), 5: (128, 128, False, 0), 6: (256, 128, False, 0), 7: (256, 256, False, 0)}


@pytest.mark.parametrize("shape,stages", [(0, 2), (0, 8), (1, 4), (2, 3), (3, 4), (4, 3), (5, 3), (6, 2), (7, 2)])
@pytest.mark.parametrize("m,n,k,ranges", [(64, 512, 1024, 1), (17, 200, 192, 2), (40, 4096, 4096, 8), (97, 72, 64, 1),
                                          (256, 520, 1024, 3), (150, 200, 320, 1), (300, 136, 2048, 5), (700, 1000, 576, 1)])
def test_the_lds_tiled_product_in_every_form(hip, m, n, k, ranges, shape, stages):
    """Every tile shape of the LDS-tiled kernel (the four multiplying waves fed by a fifth, or
    fetching for themselves), few and many stages, unsplit and split over k, plain (with a bias),
    gated, as float and as partial sums; row and column counts that fill no tile, more rows than a
    tile holds (the grid's third dimension), a k range shorter than the ring."""
    from nano_vllm_amd.kernels import KernelError
    kern = hip[torch.bfloat16]
    x, w = _rand((m, k), torch.bfloat16, 43), _rand((n, k), torch.bfloat16, 44, 0.05)
    b = _rand((n,), torch.bfloat16, 45)
    want = x.double() @ w.double().T
    kern.tile_shape = (shape, stages, ranges)
    try:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
        kern._linear_tile(x, k, w, k, b, out, n, False, False, m, n, k)
        _close(out, (want + b.double()).float().to(torch.bfloat16), torch.bfloat16)
        out32 = torch.empty((m, n), dtype=torch.float32, device=DEV)
        kern._linear_tile(x, k, w, k, None, out32, n, True, False, m, n, k)
        _close(out32, want.float(), torch.float32)
        got = kern._linear_tile(x, k, w, k, b, None, 0, False, False, m, n, k, defer=True)
        assert (ranges > 1) == hasattr(got, "tensor")
        _close(got.tensor() if hasattr(got, "tensor") else got, (want + b.double()).float().to(torch.bfloat16), torch.bfloat16)
        if ranges == 1:
            gated = torch.empty((m, n // 2), dtype=torch.bfloat16, device=DEV)
            y = want.float().to(torch.bfloat16).float()
            if shape == 0:                       # one column block per wave: no place for a gate and its up
                with pytest.raises(KernelError, match="two column blocks"):
                    kern._linear_tile(x, k, w, k, None, gated, n // 2, False, True, m, n, k)
            else:
                kern._linear_tile(x, k, w, k, None, gated, n // 2, False, True, m, n, k)
                _close(gated, (torch.nn.functional.silu(y[:, :n // 2]) * y[:, n // 2:]).to(torch.bfloat16), torch.bfloat16)
    finally:
        kern.tile_shape = None
    kern.check_faults()


def test_the_lds_tiled_product_refuses_what_it_does_not_take(hip):
    from nano_vllm_amd.kernels import KernelError
    kern = hip[torch.bfloat16]
    assert not kern._tile_takes(None, 4104, None, 4104, 32, 512, 4104)          # k no multiple of 64
    assert not kern._tile_takes(None, 4096, None, 4096, 32, 600000, 4096)       # a weight beyond 32-bit offsets
    x, w = _rand((32, 4104), torch.bfloat16, 46), _rand((9000, 4104), torch.bfloat16, 47, 0.05)
    assert kern._own_kernel(32, 9000, 4104) is None
    _close(kern.linear(x, w), (x.double() @ w.double().T).float().to(torch.bfloat16), torch.bfloat16)
    kern.tile_shape = (3, 8, 1)                  # eight stages of the largest tile: more than LDS holds
    try:
        with pytest.raises(KernelError, match="do not fit LDS"):
            kern._linear_tile(_rand((32, 128), torch.bfloat16, 48), 128, _rand((64, 128), torch.bfloat16, 49), 128, None,
                              torch.empty((32, 64), dtype=torch.bfloat16, device=DEV), 64, False, False, 32, 64, 128)
    finally:
        kern.tile_shape = None
    # the rule sends a wide weight's rows 17 to 256 to this kernel, plain, gated and as float logits
    n, k = 9216, 512
    assert n > kern.medium_max_weight_rows and kern._own_kernel(100, n, k) == "tile"
    x, w = _rand((100, k), torch.bfloat16, 50), _rand((n, k), torch.bfloat16, 51, 0.05)
    want = x.double() @ w.double().T
    _close(kern.linear(x, w), want.float().to(torch.bfloat16), torch.bfloat16)
    _close(kern.linear(x, w, out_float32=True), want.float(), torch.float32)
    y = want.float().to(torch.bfloat16).float()
    _close(kern.linear_silu_mul(x, w), (torch.nn.functional.silu(y[:, :n // 2]) * y[:, n // 2:]).to(torch.bfloat16), torch.bfloat16)
    kern.check_faults()


def test_the_kernel_for_medium_row_counts_spreads_a_weight_evenly_over_the_cus(hip):
    """What _medium_shape picks: for the gate/up weight of an 8B model (1536 blocks of 16 rows) six
    blocks a workgroup, which is one workgroup for each of 256 CUs, not eight (192 workgroups, a
    quarter of the CUs idle); a weight of few blocks is split over k until every CU has a workgroup."""
    kern = hip[torch.bfloat16]
    old = kern.medium_target_workgroups
    kern.medium_target_workgroups = 256
    try:
        waves, rt, splits = kern._medium_shape(64, 1536, 4096)
        assert waves * rt == 6 and splits == 1
        waves, rt, splits = kern._medium_shape(64, 256, 4096)
        assert (256 // (waves * rt)) * splits == 256
        assert kern._medium_shape(64, 3200, 5120) == (4, 2, 1)      # few large workgroups read x less often than many small
        assert kern._medium_shape(240, 1536, 4096) == (4, 1, 1) and kern._medium_shape(200, 3200, 5120)[:2] == (4, 2)
    finally:
        kern.medium_target_workgroups = old


def test_rotation_refuses_a_position_beyond_its_table(hip, ref):
    from nano_vllm_amd.kernels import KernelError
    k = hip[torch.float32]
    table = ref.rotary_table(_inv_freq(16, 1e4), 100)
    qkv = _rand((2, 4 * 16), torch.float32, 1)
    positions = torch.tensor([3, 100], dtype=torch.int32, device=DEV)
    with pytest.raises(KernelError, match="no row in the rotary table of 100"):
        k.qk_norm_rope_store(qkv, 2, 1, 16, None, None, 1e-6, table, positions, None, None, None, max_position=101)
    with pytest.raises(KernelError, match="needs max_position"):
        k.qk_norm_rope_store(qkv, 2, 1, 16, None, None, 1e-6, table, positions, None, None, None)


def test_split_products_are_consumed_by_norm_and_qk_kernels(hip, ref):
    """A product left as partial sums gives, through the kernels that take it, bit for bit what the
    finished product gives."""
    from nano_vllm_amd.kernels.ops import SplitSum
    k = hip[torch.bfloat16]
    m, kk = 5, 4096
    x = _rand((m, kk), torch.bfloat16, 30)
    # output projection -> fused residual sum and norm
    w = _rand((256, kk), torch.bfloat16, 31, 0.05)
    y = k.linear(x, w, deferred=True)
    assert isinstance(y, SplitSum) and y.splits > 1
    done = k.linear(x, w)
    assert torch.equal(y.tensor(), done)
    res = _rand((m, 256), torch.bfloat16, 32)
    nw = _rand((256,), torch.bfloat16, 33) + 1
    r1, r2 = res.clone(), res.clone()
    a, _ = k.add_rms_norm(y, r1, nw, 1e-6)
    b, _ = k.add_rms_norm(done, r2, nw, 1e-6)
    assert torch.equal(a, b) and torch.equal(r1, r2)
    assert torch.equal(k.rms_norm(y, nw, 1e-6), k.rms_norm(done, nw, 1e-6))
    # packed q/k/v projection with a bias -> norm, rotation and cache write
    hq, hkv, D, page = 6, 2, 64, 16
    wq = _rand(((hq + 2 * hkv) * D, kk), torch.bfloat16, 34, 0.05)
    bias = _rand(((hq + 2 * hkv) * D,), torch.bfloat16, 35)
    qkv = k.linear(x, wq, bias, deferred=True)
    assert isinstance(qkv, SplitSum)
    full = k.linear(x, wq, bias)
    table = ref.rotary_table(_inv_freq(D, 1e4), 100)
    positions = torch.tensor([3, 50, 7, 99, 0], dtype=torch.int32, device=DEV)
    slots = torch.tensor([17, 2, 40, -1, 33], dtype=torch.int32, device=DEV)
    qn, kn = _rand((D,), torch.bfloat16, 36) + 1, _rand((D,), torch.bfloat16, 37) + 1
    caches = [new_caches(4, hkv, D, page, torch.bfloat16, DEV) for _ in range(2)]
    q1 = k.qk_norm_rope_store(qkv, hq, hkv, D, qn, kn, 1e-6, table, positions, slots, *caches[0], max_position=int(positions.max()) + 1)
    q2 = k.qk_norm_rope_store(full, hq, hkv, D, qn, kn, 1e-6, table, positions, slots, *caches[1], max_position=int(positions.max()) + 1)
    assert torch.equal(q1, q2) and torch.equal(caches[0][0], caches[1][0]) and torch.equal(caches[0][1], caches[1][1])
    assert float(caches[0][1].abs().sum()) > 0
    # the same for a product of more rows, which the kernel for medium row counts leaves
    x = _rand((40, kk), torch.bfloat16, 38)
    y = k.linear(x, w, deferred=True)
    assert isinstance(y, SplitSum) and y.splits > 1
    done = k.linear(x, w)
    assert torch.equal(y.tensor(), done)
    assert torch.equal(k.rms_norm(y, nw, 1e-6), k.rms_norm(done, nw, 1e-6))


def test_library_products_are_run_by_the_norm_that_adds_them(hip):
    """A product of many rows handed to the residual norm is run there, the sum in the product's
    epilogue: residual + x W^T in float rounded once, then the norm of that; every other
    consumer gets the plain product."""
    from nano_vllm_amd.kernels.ops import PendingProduct
    k = hip[torch.bfloat16]
    m, kk, n = 300, 1024, 768
    x = _rand((m, kk), torch.bfloat16, 40)
    w = _rand((n, kk), torch.bfloat16, 41, 0.05)
    res = _rand((m, n), torch.bfloat16, 42)
    nw = _rand((n,), torch.bfloat16, 43) + 1
    y = k.linear(x, w, deferred=True)
    assert isinstance(y, PendingProduct) and y.shape == (m, n)
    assert torch.equal(y.tensor(), k.linear(x, w))
    assert torch.equal(k.rms_norm(y, nw, 1e-6), k.rms_norm(k.linear(x, w), nw, 1e-6))
    r = res.clone()
    a, r_out = k.add_rms_norm(k.linear(x, w, deferred=True), r, nw, 1e-6)
    assert r_out is r
    want_r = x.double() @ w.double().t() + res.double()
    _close(r, want_r, torch.bfloat16, "residual + product")
    assert torch.equal(a, k.rms_norm(r, nw, 1e-6))
    # the sum is rounded once: closer to the exact sum than product and sum rounded in turn
    two = (k.linear(x, w).float() + res.float()).bfloat16()
    assert float((r.double() - want_r).abs().mean()) <= float((two.double() - want_r).abs().mean())
    # with a bias, or a result that is asked for as a tensor, nothing is left pending
    bias = _rand((n,), torch.bfloat16, 44)
    assert isinstance(k.linear(x, w, bias, deferred=True), torch.Tensor)
    assert isinstance(k.linear(x, w), torch.Tensor)
    with pytest.raises(Exception, match="residual does not match"):
        k.add_rms_norm(k.linear(x, w, deferred=True), res[:10].clone(), nw, 1e-6)


# ------------------------------------------------------------------------------ rotation and cache write
def _inv_freq(D, theta):
    return (1.0 / (theta ** (torch.arange(0, D, 2, dtype=torch.float) / D))).to(DEV)


@pytest.mark.parametrize("D,theta,P", [(16, 1e4, 128), (48, 5e5, 300), (128, 1e6, 4096)])
def test_rotary_table(hip, D, theta, P):
    inv = _inv_freq(D, theta)
    t = hip[torch.float32].rotary_table(inv, P)
    ang = plain.rope_angles(D, torch.arange(P), theta)                # the reference's float32 angles, on the CPU
    assert float((t[:, : D // 2].cpu() - ang.cos()).abs().max()) < 2e-6
    assert float((t[:, D // 2:].cpu() - ang.sin()).abs().max()) < 2e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,D,page,norm", [(4, 2, 16, 4, True), (5, 5, 48, 16, True), (6, 2, 64, 8, False),
                                                 (7, 1, 80, 64, True), (8, 2, 128, 256, True), (3, 3, 256, 32, True)])
def test_qk_norm_rope_store(hip, ref, dtype, hq, hkv, D, page, norm):
    T = 37
    pages = (T + page - 1) // page + 2
    k = hip[dtype]
    qkv = _rand((T, (hq + 2 * hkv) * D), dtype, 17)
    qw = _rand((D,), dtype, 18) + 1 if norm else None
    kw = _rand((D,), dtype, 19) + 1 if norm else None
    table = ref.rotary_table(_inv_freq(D, 1e4), 500)
    positions = torch.randint(0, 500, (T,), dtype=torch.int32, device=DEV)
    slots = torch.randperm(pages * page)[:T].to(torch.int32).to(DEV)
    slots[5] = -1                                                   # this token is not stored
    caches = [new_caches(pages, hkv, D, page, dtype, DEV) for _ in range(2)]
    a, b = qkv.clone(), qkv.clone()
    qa = k.qk_norm_rope_store(a, hq, hkv, D, qw, kw, 1e-6, table, positions, slots, *caches[0], max_position=int(positions.max()) + 1)
    qb = ref.qk_norm_rope_store(b, hq, hkv, D, qw, kw, 1e-6, table, positions, slots, *caches[1], max_position=int(positions.max()) + 1)
    _close(qa, qb, dtype, "q")
    _close(a, b, dtype, "k in place")
    _close(caches[0][0], caches[1][0], dtype, "k cache")
    assert torch.equal(caches[0][1], caches[1][1])                  # values are copied as they are
    assert float(caches[0][0].abs().sum()) > 0
    # without norm weights and table the kernel only stores
    c = qkv.clone()
    k.qk_norm_rope_store(c, hq, hkv, D, None, None, 1e-6, None, None, slots, *caches[0])
    assert torch.equal(c, qkv)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,D,page", [(4, 2, 16, 8), (3, 1, 32, 32), (6, 2, 64, 64), (8, 2, 128, 256),
                                           (2, 2, 256, 32), (5, 5, 48, 16), (4, 1, 128, 24)])
def test_qk_norm_rope_store_of_a_long_portion(hip, ref, dtype, hq, hkv, D, page):
    """Many tokens take the tiled kernel: slots in a row from the start of a key tile (written
    eight keys at a time), slots in a row from the middle of one, scattered slots, tokens that
    are not stored, and a last block that is not full."""
    T = 331
    pages = (T + 416 + page - 1) // page + 6                        # slots 0..415 hold the runs
    k = hip[dtype]
    qkv = _rand((T, (hq + 2 * hkv) * D), dtype, 41)
    qw, kw = _rand((D,), dtype, 42) + 1, _rand((D,), dtype, 43) + 1
    table = ref.rotary_table(_inv_freq(D, 1e6), 700)
    positions = torch.randint(0, 700, (T,), dtype=torch.int32, device=DEV)
    slots = torch.randperm(pages * page - 416)[:T] + 416            # scattered, beyond the runs
    slots[0:128] = torch.arange(128, 256)                           # in a row from the start of a tile
    slots[128:230] = torch.arange(5, 5 + 102)                       # in a row from the middle of a tile
    slots[256:320] = torch.arange(256 + 96, 256 + 160)              # another run that starts at a tile
    slots[17] = -1
    slots[300] = -1
    slots = slots.to(torch.int32).to(DEV)
    assert len(set(slots.tolist()) - {-1}) == T - 2
    caches = [new_caches(pages, hkv, D, page, dtype, DEV) for _ in range(2)]
    a, b = qkv.clone(), qkv.clone()
    qa = k.qk_norm_rope_store(a, hq, hkv, D, qw, kw, 1e-6, table, positions, slots, *caches[0], max_position=int(positions.max()) + 1)
    qb = ref.qk_norm_rope_store(b, hq, hkv, D, qw, kw, 1e-6, table, positions, slots, *caches[1], max_position=int(positions.max()) + 1)
    _close(qa, qb, dtype, "q")
    _close(a, b, dtype, "k in place")
    _close(caches[0][0], caches[1][0], dtype, "k cache")
    assert torch.equal(caches[0][1], caches[1][1])                  # values are copied as they are
    assert torch.equal(a[:, (hq + hkv) * D:], qkv[:, (hq + hkv) * D:])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,D,rot,page,T", [(4, 2, 16, 8, 4, 37), (5, 5, 48, 16, 16, 37), (8, 2, 128, 64, 256, 100),
                                                  (3, 1, 80, 30, 64, 70), (2, 2, 256, 2, 32, 9), (7, 1, 64, 62, 8, 37)])
def test_qk_norm_rope_store_with_a_rotation_of_fewer_channels(hip, ref, dtype, hq, hkv, D, rot, page, T):
    """A table narrower than the head: the first `rot` channels are rotated in pairs (i, i + rot/2)
    by the angles of a head of that size, the others are only normed.  Checked against the stand-in
    and, channel by channel, against the plain rotation of the slice."""
    pages = (T + page - 1) // page + 2
    k = hip[dtype]
    qkv = _rand((T, (hq + 2 * hkv) * D), dtype, 51)
    qw, kw = _rand((D,), dtype, 52) + 1, _rand((D,), dtype, 53) + 1
    table = ref.rotary_table(_inv_freq(rot, 1e4), 500)
    assert table.shape == (500, rot)
    positions = torch.randint(0, 500, (T,), dtype=torch.int32, device=DEV)
    slots = torch.randperm(pages * page)[:T].to(torch.int32).to(DEV)
    caches = [new_caches(pages, hkv, D, page, dtype, DEV) for _ in range(2)]
    a, b = qkv.clone(), qkv.clone()
    qa = k.qk_norm_rope_store(a, hq, hkv, D, qw, kw, 1e-6, table, positions, slots, *caches[0], max_position=500)
    qb = ref.qk_norm_rope_store(b, hq, hkv, D, qw, kw, 1e-6, table, positions, slots, *caches[1], max_position=500)
    _close(qa, qb, dtype, "q")
    _close(a, b, dtype, "k in place")
    _close(caches[0][0], caches[1][0], dtype, "k cache")
    assert torch.equal(caches[0][1], caches[1][1])
    # without norm weights: the channels from rot on come back as they were, and the first rot are
    # the plain rotation of that slice
    c = qkv.clone()
    qc = k.qk_norm_rope_store(c, hq, hkv, D, None, None, 1e-6, table, positions, None, None, None, max_position=500)
    heads = qkv[:, : hq * D].reshape(T, hq, D)
    got = qc.reshape(T, hq, D)
    assert torch.equal(got[..., rot:], heads[..., rot:])
    ang = plain.rope_angles(rot, positions.cpu(), 1e4)
    want = plain.apply_rope(heads[..., :rot].float().cpu(), ang)
    _close(got[..., :rot].cpu(), want.to(dtype), dtype, "rotated slice")
    # partial sums take the same kernel
    if dtype == torch.bfloat16:
        from nano_vllm_amd.kernels.ops import SplitSum
        width = (hq + 2 * hkv) * D
        sums = torch.stack([qkv.float() * 0.75, qkv.float() * 0.25])
        part = SplitSum(k, sums.reshape(-1), 2, T, width, None)
        assert torch.equal(part.tensor(), qkv)
        caches2 = new_caches(pages, hkv, D, page, dtype, DEV)
        qp = k.qk_norm_rope_store(part, hq, hkv, D, qw, kw, 1e-6, table, positions, slots, *caches2, max_position=500)
        assert torch.equal(qp, qa) and torch.equal(caches2[0], caches[0][0]) and torch.equal(caches2[1], caches[0][1])


def test_qk_refusals(hip):
    from nano_vllm_amd.kernels import KernelError
    k = hip[torch.float32]
    with pytest.raises(KernelError, match="width"):
        k.qk_norm_rope_store(torch.zeros((2, 100), device=DEV), 2, 1, 16, None, None, 1e-6, None, None, None, None, None)
    with pytest.raises(KernelError, match="head_dim"):
        k.qk_norm_rope_store(torch.zeros((2, 4 * 1024), device=DEV), 2, 1, 1024, None, None, 1e-6, None, None, None, None, None)
    positions = torch.zeros(2, dtype=torch.int32, device=DEV)
    for width in (18, 7):                                          # wider than the head; odd
        with pytest.raises(KernelError, match="rot even and at most"):
            k.qk_norm_rope_store(torch.zeros((2, 4 * 16), device=DEV), 2, 1, 16, None, None, 1e-6,
                                 torch.zeros((10, width), device=DEV), positions, None, None, None, max_position=1)


# ------------------------------------------------------------------------------ attention
def _paged_case(dtype, hq, hkv, D, page, lens, q_lens, seed, boost=None, fill=1.0):
    """A batch of requests with kv lengths `lens`, the last q_lens of which are this step's
    queries; keys and values scattered over shuffled pages."""
    rng = random.Random(seed)
    S = len(lens)
    pages_per = [(n + page - 1) // page for n in lens]
    total = sum(pages_per) + 3
    order = list(range(total))
    rng.shuffle(order)
    kc, vc = new_caches(total, hkv, D, page, dtype, DEV, fill=None if math.isnan(fill) else fill)
    if math.isnan(fill):                                            # what unused slots hold must not matter
        kc.fill_(fill), vc.fill_(fill)
    vt = vc.shape[4]
    width = max(pages_per)
    tables = torch.full((S, width), -1, dtype=torch.int32)
    ks, vs, qs, token_seq, positions = [], [], [], [], []
    for s, n in enumerate(lens):
        mine = [order.pop() for _ in range(pages_per[s])]
        tables[s, : len(mine)] = torch.tensor(mine, dtype=torch.int32)
        k = _rand((n, hkv, D), dtype, seed * 100 + s)
        v = _rand((n, hkv, D), dtype, seed * 100 + 50 + s)
        q = _rand((n, hq, D), dtype, seed * 100 + 70 + s)
        if boost is not None:                                       # one far key that every late query prefers
            k[boost] = 0
            k[boost, :, 0] = 8.0                                    # score 64; every other key: 8 * N(0, 1)
            q[:] = 0
            q[:, :, 0] = 8.0
        for j in range(n):
            kc[mine[j // page], :, j % page, :] = k[j]
            vc[mine[j // page], :, (j % page) // vt, :, (j % page) % vt] = v[j]
        ks.append(k); vs.append(v); qs.append(q)
        token_seq += [s] * q_lens[s]
        positions += list(range(n - q_lens[s], n))
    q = torch.cat([qs[s][lens[s] - q_lens[s]:] for s in range(S)]).reshape(sum(q_lens), hq * D).contiguous()
    batch = SimpleNamespace(
        num_seqs=S, num_tokens=sum(q_lens), token_seq=torch.tensor(token_seq, dtype=torch.int32, device=DEV),
        positions=torch.tensor(positions, dtype=torch.int32, device=DEV), max_kv_len=max(lens), max_q_len=max(q_lens),
        kv_lens=torch.tensor(lens, dtype=torch.int32, device=DEV),
        cu_seqlens_q=torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=DEV),
        num_decode=next((i for i, n in enumerate(q_lens) if n != 1), len(q_lens)), q_lens=list(q_lens),
        groups=[SimpleNamespace(block_tables=tables.to(DEV), slot_mapping=None)])
    return q, kc, vc, batch, (qs, ks, vs)


def _plain_attention(qs, ks, vs, lens, q_lens, scale, window=None):
    out = []
    for q, k, v, n, nq in zip(qs, ks, vs, lens, q_lens):
        o = plain.causal_attention(q.float().cpu(), k.float().cpu(), v.float().cpu(), scale, window)
        out.append(o[n - nq:].reshape(nq, -1))
    return torch.cat(out)


ATT_CASES = [
    # hq, hkv, D, page, kv lens, q lens, window
    (4, 2, 16, 4, [5, 11, 17], [5, 11, 17], None),                 # whole prompts
    (8, 2, 32, 8, [40, 9, 24, 3], [1, 1, 16, 3], None),            # decode beside portions
    (6, 3, 48, 16, [100, 33], [1, 20], None),
    (5, 5, 80, 64, [130, 64, 65], [2, 64, 1], None),               # page edges
    (8, 2, 128, 256, [700, 300, 257], [1, 1, 1], None),            # long decode
    (7, 1, 64, 32, [90, 31], [45, 1], None),                       # seven heads on one kv head
    (4, 2, 128, 16, [200, 50], [30, 1], 24),                       # window
    (2, 1, 256, 8, [33], [33], 5),
    (8, 2, 128, 64, [300, 500, 77, 130], [1, 1, 77, 100], None),   # the shape of a served step
    (4, 4, 64, 16, [1, 2, 3, 40], [1, 2, 3, 40], None),            # the first tokens of requests
    (16, 1, 32, 8, [70, 9], [1, 9], None),                         # sixteen heads on one kv head
    (3, 1, 96, 24, [150, 100], [1, 100], 40),                      # a window over pages of 24
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,D,page,lens,q_lens,window", ATT_CASES)
def test_paged_attention(hip, ref, dtype, hq, hkv, D, page, lens, q_lens, window):
    q, kc, vc, batch, parts = _paged_case(dtype, hq, hkv, D, page, lens, q_lens, seed=3)
    scale = D ** -0.5
    got = hip[dtype].paged_attention(q, hq, hkv, D, kc, vc, batch, 0, scale, window)
    want = _plain_attention(*parts, lens, q_lens, scale, window).to(DEV)
    _close(got, want.to(dtype), dtype, "against the plain whole-sequence attention")
    twin = ref.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, scale, window)
    _close(got, twin, dtype, "against the plain paged attention")
    hip[dtype].check_faults()
    if dtype == torch.bfloat16:
        # the general kernel in bfloat16 (the fallback of shapes the matrix-core kernels refuse)
        hip[dtype].mfma_attention = False
        try:
            _close(hip[dtype].paged_attention(q, hq, hkv, D, kc, vc, batch, 0, scale, window), twin, dtype, "general")
        finally:
            hip[dtype].mfma_attention = True


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,D,page,lens,q_lens", [case[:6] for case in ATT_CASES if case[6] is None and case[2] <= 128] + [
    (4, 2, 128, 256, [700, 90, 300], [1, 90, 257], ),              # a single token, a whole prompt, a portion behind 43 keys
    (3, 3, 40, 8, [77, 130], [33, 130]),                           # a head size that is no multiple of 8
    (2, 1, 112, 24, [100], [64]),
])
def test_general_attention_of_portions_gives_the_bits_of_one_wave_per_token(hip, dtype, hq, hkv, D, page, lens, q_lens):
    """The general kernel has a form for portions of prompts that stages the keys once for 32 rows; its
    arithmetic is the per-token kernel's, so the results are equal bit for bit, unused cache slots
    holding no numbers."""
    q, kc, vc, batch, parts = _paged_case(dtype, hq, hkv, D, page, lens, q_lens, seed=13, fill=float("nan"))
    k, scale = hip[dtype], D ** -0.5
    k.mfma_attention = False
    try:
        tiled = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, scale, None)
        k.tiled_general_attention = False
        per_token = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, scale, None)
    finally:
        k.mfma_attention = k.tiled_general_attention = True
    k.check_faults()
    assert torch.equal(tiled, per_token)
    _close(tiled, _plain_attention(*parts, lens, q_lens, scale, None).to(DEV).to(dtype), dtype)


@pytest.mark.parametrize("sets", [1, 2])
@pytest.mark.parametrize("hq,hkv,D,page,lens,q_lens,window", [
    (8, 2, 128, 256, [700, 1300], [700, 900], None),               # pages of whole tiles: the run of whole tiles
    (8, 2, 128, 64, [1100, 130], [300, 130], None),                # a portion after a prefix, a page a tile
    (4, 1, 64, 128, [900], [900], 200),                            # a window: tiles cut at both ends
    (6, 2, 96, 24, [333, 80], [333, 1], None),                     # pages that hold no whole tile
    (3, 3, 32, 8, [150], [150], 70),
    (2, 1, 256, 64, [400], [250], None),                           # one wave per SIMD: always one set
    (5, 1, 160, 32, [130, 70], [130, 70], None),                   # five heads: a second chunk with one wave at work
])
def test_prefill_attention_with_one_and_two_sets_of_waves(hip, sets, hq, hkv, D, page, lens, q_lens, window):
    """The matrix-core prefill kernel with its waves as one set and as two (the launcher's own choice
    goes by the number of workgroups), against the plain whole-sequence attention; what the cache
    holds where no key was written is not a number."""
    from nano_vllm_amd.kernels import library
    dtype = torch.bfloat16
    q, kc, vc, batch, parts = _paged_case(dtype, hq, hkv, D, page, lens, q_lens, seed=11, fill=float("nan"))
    scale = D ** -0.5
    want = _plain_attention(*parts, lens, q_lens, scale, window).to(DEV)
    lib = library.load("attn_prefill", "bf16")
    lib.nva_attn_prefill_sets(sets)
    try:
        got = hip[dtype].paged_attention(q, hq, hkv, D, kc, vc, batch, 0, scale, window)
    finally:
        lib.nva_attn_prefill_sets(-1)
    _close(got, want.to(dtype), dtype, f"{sets} sets")
    hip[dtype].check_faults()


@pytest.mark.parametrize("page", [64, 256, 24])
def test_prefill_attention_behind_a_window_whose_first_pages_were_given_back(hip, page):
    """A portion late in a long request behind a window: the block table has no page (-1) where no
    row sees a key any more, the kernel reads page 0 for such entries, and page 0 holds no numbers."""
    dtype, hq, hkv, D, window = torch.bfloat16, 4, 2, 128, 300
    lens, q_lens = [1500], [200]
    q, kc, vc, batch, parts = _paged_case(dtype, hq, hkv, D, page, lens, q_lens, seed=17, fill=float("nan"))
    tables = batch.groups[0].block_tables
    # page 0 is made free: what it holds moves to a page nobody uses, which the table then names
    used = set(tables.flatten().tolist())
    spare = next(i for i in range(kc.shape[0]) if i not in used and i != 0)
    kc[spare], vc[spare] = kc[0], vc[0]
    tables[tables == 0] = spare
    kc[0], vc[0] = float("nan"), float("nan")
    first_seen = lens[0] - q_lens[0] - window + 1                  # the first key the portion's first row sees
    tables[0, : first_seen // page] = -1
    scale = D ** -0.5
    want = _plain_attention(*parts, lens, q_lens, scale, window).to(DEV)
    got = hip[dtype].paged_attention(q, hq, hkv, D, kc, vc, batch, 0, scale, window)
    _close(got, want.to(dtype), dtype, f"page {page}")
    hip[dtype].check_faults()


@pytest.mark.parametrize("seed", range(12))
def test_attention_of_drawn_shapes(hip, ref, seed):
    """Head counts, groups, head sizes, page sizes, windows and lengths drawn at random (single tokens
    first, as the engine orders a step): the bfloat16 kernels against the plain whole-sequence attention."""
    rng = random.Random(1000 + seed)
    hkv = rng.choice([1, 2, 3, 5])
    G = rng.choice([1, 2, 3, 4, 7, 8, 16])
    D = rng.choice([32, 64, 96, 128, 160, 256])
    page = rng.choice([8, 16, 24, 64])
    window = rng.choice([None, None, 5, 33, 100])
    decodes = rng.randint(1, 12)
    lens = [rng.randint(1, 300) for _ in range(decodes)]
    q_lens = [1] * decodes
    for _ in range(rng.randint(0, 2)):
        n = rng.randint(2, 200)
        lens.append(n + rng.choice([0, 0, rng.randint(1, 150)]))
        q_lens.append(n)
    dtype = torch.bfloat16
    q, kc, vc, batch, parts = _paged_case(dtype, hkv * G, hkv, D, page, lens, q_lens, seed=200 + seed)
    scale = D ** -0.5
    got = hip[dtype].paged_attention(q, hkv * G, hkv, D, kc, vc, batch, 0, scale, window)
    want = _plain_attention(*parts, lens, q_lens, scale, window).to(DEV)
    _close(got, want.to(dtype), dtype, f"hkv {hkv} group {G} head_dim {D} page {page} window {window} lens {lens} q {q_lens}")
    hip[dtype].check_faults()


@pytest.mark.parametrize("seed", range(10))
def test_products_of_drawn_shapes(hip, ref, seed):
    """Rows, widths and depths drawn at random over the ranges of the weight-streaming kernels (k a
    multiple of 8, anything else free), plain, with a bias, with a float result, left as partial sums."""
    from nano_vllm_amd.kernels.ops import SplitSum
    rng = random.Random(2000 + seed)
    m = rng.choice([rng.randint(1, 16), rng.randint(17, 128), rng.randint(129, 256)])
    n = rng.choice([rng.randint(1, 300), rng.randint(1000, 9000)])
    k = 8 * rng.choice([rng.randint(1, 40), rng.randint(100, 700)])
    kern = hip[torch.bfloat16]
    x, w = _rand((m, k), torch.bfloat16, 3000 + seed), _rand((n, k), torch.bfloat16, 3100 + seed, 0.05)
    b = _rand((n,), torch.bfloat16, 3200 + seed)
    want = x.double() @ w.double().T
    what = f"m {m} n {n} k {k}"
    _close(kern.linear(x, w), want.float().to(torch.bfloat16), torch.bfloat16, what)
    _close(kern.linear(x, w, b), (want + b.double()).float().to(torch.bfloat16), torch.bfloat16, what + " with a bias")
    bound = (x.double().abs() @ w.double().abs().T) * (math.sqrt(k) * 2.0 ** -23) + 1e-30
    assert bool(((kern.linear(x, w, out_float32=True).double() - want).abs() <= bound).all()), what + " float result"
    y = kern.linear(x, w, b, deferred=True)
    if isinstance(y, SplitSum):
        assert torch.equal(y.tensor(), kern.linear(x, w, b)), what + " deferred"
    kern.check_faults()


@pytest.mark.parametrize("seed", range(12))
def test_the_lds_tiled_product_at_drawn_shapes(hip, seed):
    """Rows, widths, depths (multiples of 64), tile shapes, stages and cuts of k drawn at random for
    the LDS-tiled kernel: plain with a bias, float within the bound of its rounding, gated, and
    the partial sums added up."""
    rng = random.Random(5000 + seed)
    shape = rng.randrange(8)
    bm, bn, fed, sx = TILE_SHAPES[shape]
    lds = lambda st: (sx * bm + st * bn) * 128 if fed else st * (bm + bn) * 128
    stages = rng.choice([st for st in ((2, 3, 4, 8) if fed else (2, 3)) if lds(st) <= 160 * 1024])
    m = rng.choice([rng.randint(17, 64), rng.randint(65, 256), rng.randint(257, 600)])
    n = 2 * rng.choice([rng.randint(1, 150), rng.randint(500, 4500)])
    k = 64 * rng.choice([rng.randint(1, 8), rng.randint(20, 90)])
    ranges = rng.choice([1, 1, rng.randint(2, 9)])
    # columns of the result per workgroup: the whole tile, or fewer (a multiple of 8 as the engine
    # draws them, or any number); the gated form's tile has half as many columns as rows of W
    cols = rng.choice([0, 0, 8 * rng.randint(1, bn // 16), rng.randint(1, bn // 2)])
    kern = hip[torch.bfloat16]
    x, w = _rand((m, k), torch.bfloat16, 5100 + seed), _rand((n, k), torch.bfloat16, 5200 + seed, 0.05)
    b = _rand((n,), torch.bfloat16, 5300 + seed)
    want = x.double() @ w.double().T
    what = f"m {m} n {n} k {k} shape {shape} stages {stages} ranges {ranges} columns {cols}"
    kern.tile_shape = (shape, stages, ranges, cols)
    try:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
        kern._linear_tile(x, k, w, k, b, out, n, False, False, m, n, k)
        _close(out, (want + b.double()).float().to(torch.bfloat16), torch.bfloat16, what)
        out32 = torch.empty((m, n), dtype=torch.float32, device=DEV)
        kern._linear_tile(x, k, w, k, None, out32, n, True, False, m, n, k)
        bound = (x.double().abs() @ w.double().abs().T) * (math.sqrt(k) * 2.0 ** -23) + 1e-30
        assert bool(((out32.double() - want).abs() <= bound).all()), what + " float result"
        got = kern._linear_tile(x, k, w, k, None, None, 0, False, False, m, n, k, defer=True)
        if hasattr(got, "tensor"):
            sums = got.sums[:got.splits * m * n].view(got.splits, m, n).double().sum(0)
            assert bool(((sums - want).abs() <= bound).all()), what + " partial sums"
        if shape != 0:
            kern.tile_shape = (shape, stages, 1, cols)
            gated = torch.empty((m, n // 2), dtype=torch.bfloat16, device=DEV)
            kern._linear_tile(x, k, w, k, None, gated, n // 2, False, True, m, n, k)
            y = want.float().to(torch.bfloat16).float()
            _close(gated, (torch.nn.functional.silu(y[:, :n // 2]) * y[:, n // 2:]).to(torch.bfloat16), torch.bfloat16, what + " gated")
    finally:
        kern.tile_shape = None
    kern.check_faults()


@pytest.mark.parametrize("page,lens,q_lens,window", [
    (256, [40000, 12345, 257, 4096], [1, 1, 1, 1], None),           # long decoding: 157 pages in a table
    (16, [30000, 5000], [1, 1], None),                              # the same over small pages: splits capped by pages
    (256, [9000, 20000], [1, 700], None),                           # a portion after a long cached prefix
    (64, [33000], [1500], 4096),                                    # a window far into a long request
    (256, [16000, 16000, 16000], [1, 1, 300], 1000),
])
def test_attention_over_long_contexts_against_plain_arithmetic(hip, page, lens, q_lens, window):
    """Tens of thousands of keys: the bfloat16 matrix-core kernels (decode with splits, prefill
    with its block table in LDS) and the general kernel, each against a float softmax over the
    keys and values gathered from the pages.  The cache is filled directly; the tables are a
    random permutation."""
    _kernels_against_gathered_attention(hip, page, lens, q_lens, window)


@pytest.mark.parametrize("page,count,longest,window,seed", [
    (64, 1100, 300, None, 1),       # more single tokens than one launch of the decode kernel takes
    (16, 300, 700, 37, 2),          # many requests of very different lengths behind a window
    (256, 200, 3000, None, 3),      # a wave's share of the keys spans several requests, and a request several waves
    (8, 40, 90, None, 4),           # requests shorter than a chunk of keys
])
def test_decode_attention_shares_the_keys_of_many_requests_out_evenly(hip, page, count, longest, window, seed):
    rng = random.Random(seed)
    lens = [rng.randint(1, longest) for _ in range(count)]
    _kernels_against_gathered_attention(hip, page, lens, [1] * count, window)


def _gathered_attention(q, kc, vc, tables, lens, q_lens, hq, hkv, D, page, scale, window):
    """Plain float attention of each request's last q_lens tokens over its keys and values, which
    are gathered from the pages its block table names (K [pages, kv heads, page, D], V in tiles
    of vt keys [pages, kv heads, page / vt, D, vt]).  Shares nothing with the kernels."""
    out, row = [], 0
    G = hq // hkv
    for s, (n, nq) in enumerate(zip(lens, q_lens)):
        pages = tables[s, : (n + page - 1) // page].long().to(kc.device)
        K = kc[pages].float().permute(1, 0, 2, 3).reshape(hkv, -1, D)[:, :n]                    # [hkv, n, D]
        V = vc[pages].float().permute(1, 0, 2, 4, 3).reshape(hkv, -1, D)[:, :n]                 # tiles -> keys
        Q = q[row:row + nq].float().view(nq, hkv, G, D).permute(1, 2, 0, 3)                      # [hkv, G, nq, D]
        scores = torch.einsum("hgqd,hkd->hgqk", Q, K) * scale
        qpos = torch.arange(n - nq, n, device=kc.device)[:, None]
        kpos = torch.arange(n, device=kc.device)[None, :]
        seen = kpos <= qpos
        if window:
            seen &= (qpos - kpos) < window
        scores = scores.masked_fill(~seen, float("-inf"))
        o = torch.einsum("hgqk,hkd->hgqd", torch.softmax(scores, dim=-1), V)                      # [hkv, G, nq, D]
        out.append(o.permute(2, 0, 1, 3).reshape(nq, hq * D))
        row += nq
    return torch.cat(out)


def _kernels_against_gathered_attention(hip, page, lens, q_lens, window):
    hq, hkv, D = 8, 2, 128
    k = hip[torch.bfloat16]
    S = len(lens)
    pages_per = [(n + page - 1) // page for n in lens]
    total = sum(pages_per) + 5
    gen = torch.Generator(device=DEV).manual_seed(77)
    kc = torch.randn((total, hkv, page, D), generator=gen, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    vc = torch.randn(v_cache_shape(total, hkv, D, page), generator=gen, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    perm = torch.randperm(total).tolist()
    tables = torch.full((S, max(pages_per)), -1, dtype=torch.int32)
    token_seq, positions = [], []
    for s_, n in enumerate(lens):
        tables[s_, :pages_per[s_]] = torch.tensor([perm.pop() for _ in range(pages_per[s_])], dtype=torch.int32)
        token_seq += [s_] * q_lens[s_]
        positions += list(range(n - q_lens[s_], n))
    assert sorted(q_lens, key=lambda n: n != 1) == list(q_lens)     # single tokens first, as the engine orders a step
    T = sum(q_lens)
    q = (torch.randn((T, hq * D), generator=gen, device=DEV, dtype=torch.float32) * 2).to(torch.bfloat16)
    batch = SimpleNamespace(
        num_seqs=S, num_tokens=T, token_seq=torch.tensor(token_seq, dtype=torch.int32, device=DEV),
        positions=torch.tensor(positions, dtype=torch.int32, device=DEV), max_kv_len=max(lens), max_q_len=max(q_lens),
        kv_lens=torch.tensor(lens, dtype=torch.int32, device=DEV),
        cu_seqlens_q=torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=DEV),
        num_decode=next((i for i, n in enumerate(q_lens) if n != 1), len(q_lens)), q_lens=list(q_lens),
        groups=[SimpleNamespace(block_tables=tables.to(DEV), slot_mapping=None)])
    want = _gathered_attention(q, kc, vc, tables, lens, q_lens, hq, hkv, D, page, D ** -0.5, window)
    got = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, D ** -0.5, window)
    _close(got, want, torch.bfloat16, "matrix-core kernels against the float softmax over gathered keys")
    k.mfma_attention = False
    try:
        general = k.paged_attention(q, hq, hkv, D, kc, vc, batch, 0, D ** -0.5, window)
    finally:
        k.mfma_attention = True
    _close(general, want, torch.bfloat16, "general kernel against the float softmax over gathered keys")
    k.check_faults()


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_reads_a_far_key_among_hundreds(hip, dtype):
    # key 3 scores far above all others for every query: the output must be its value
    hq, hkv, D, page, lens, q_lens = 4, 2, 64, 16, [600], [40]
    q, kc, vc, batch, (qs, ks, vs) = _paged_case(dtype, hq, hkv, D, page, lens, q_lens, seed=5, boost=3)
    got = hip[dtype].paged_attention(q, hq, hkv, D, kc, vc, batch, 0, 1.0, None).float()
    want = vs[0][3].float().repeat_interleave(hq // hkv, 0).reshape(1, hq * D).expand(40, -1)
    assert float((got - want).abs().max()) < 0.05
    # with a window that ends after it, the far key is gone
    got_w = hip[dtype].paged_attention(q, hq, hkv, D, kc, vc, batch, 0, 1.0, 100).float()
    assert float((got_w - want).abs().max()) > 0.5


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_window_edge(hip, dtype):
    # exactly `window` keys are seen: the key at p - window is out, the one at p - window + 1 is in
    hq, hkv, D, page, W = 2, 1, 32, 8, 16
    for boost, inside in ((83, False), (84, True)):                 # the query stands at position 99
        q, kc, vc, batch, (qs, ks, vs) = _paged_case(dtype, hq, hkv, D, page, [100], [1], seed=7, boost=boost)
        got = hip[dtype].paged_attention(q, hq, hkv, D, kc, vc, batch, 0, 1.0, W).float()
        want = vs[0][boost].float().repeat_interleave(hq, 0).reshape(1, hq * D)
        assert (float((got - want).abs().max()) < 0.05) == inside


def test_attention_flags_a_missing_page(hip):
    from nano_vllm_amd.kernels import KernelError
    q, kc, vc, batch, _ = _paged_case(torch.float32, 2, 1, 16, 4, [10], [1], seed=1)
    batch.groups[0].block_tables[0, 1] = -1
    hip[torch.float32].paged_attention(q, 2, 1, 16, kc, vc, batch, 0, 1.0, None)
    with pytest.raises(KernelError, match="page"):
        hip[torch.float32].check_faults()


# ------------------------------------------------------------------------------ sampling
def test_sampling_matches_the_plain_draw(hip):
    from nano_vllm_amd.sampling.sampler import noise_key
    k = hip[torch.float32]
    V, R = 1001, 6
    logits = _rand((R, V), torch.float32, 20, 3.0)
    logits[0, 17] = logits[0, 900] = 50.0                           # a tie: the lowest index wins
    temps = torch.tensor([0.0, 0.0, 0.7, 1.0, 0.3, 1.5], device=DEV)
    keys = torch.tensor([noise_key(9, r, 100 + r) for r in range(R)], dtype=torch.int64, device=DEV)
    got = k.sample(logits, temps, keys).tolist()
    want = [plain.sample(logits[r].cpu(), float(temps[r]), seed=9, request=r, position=100 + r) for r in range(R)]
    assert got == want and got[0] == 17


def _exact_draws(logits, temps, keys):
    """argmax(l / T - log(-log u)) in double for whole rows at once: the kernel's generator written with
    torch's 64-bit integers (multiplication wraps; the shifts are made logical by masking)."""
    def shr(z, n):
        return (z >> n) & ((1 << (64 - n)) - 1)

    def as_i64(c):
        return c - (1 << 64) if c >= (1 << 63) else c
    rows, vocab = logits.shape
    entry = torch.arange(vocab, dtype=torch.int64, device=logits.device)
    out = []
    for r in range(rows):
        z = (keys[r] ^ entry) + as_i64(0x9E3779B97F4A7C15)
        z = (z ^ shr(z, 30)) * as_i64(0xBF58476D1CE4E5B9)
        z = (z ^ shr(z, 27)) * as_i64(0x94D049BB133111EB)
        z = z ^ shr(z, 31)
        u = (shr(z, 40).double() + 0.5) / 16777216.0
        score = logits[r].double()
        if float(temps[r]) > 0:
            score = score / float(temps[r]) - torch.log(-torch.log(u))
        out.append(int(torch.argmax(score)))
    return out


def test_sampling_passes_by_no_entry_that_wins(hip):
    """The kernel takes the score of most entries in float first and passes them by when they cannot
    beat the best so far; the entry it chooses is the one the scores in double choose: rows of the
    size of a real vocabulary, temperatures from 0.01 to 50, logits that are large, flat, or equal."""
    from nano_vllm_amd.sampling.sampler import noise_key
    k = hip[torch.float32]
    V, R = 151936, 48
    logits = _rand((R, V), torch.float32, 61, 3.0)
    logits[8:16] *= 20.0                                            # large
    logits[16:24] *= 1e-3                                           # flat: the noise decides
    logits[24:28] = 1.5                                             # all equal
    logits[28:32] = -80.0 + _rand((4, V), torch.float32, 62, 1e-2)
    temps = torch.tensor([[0.01, 0.1, 0.6, 1.0, 2.0, 7.0, 50.0, 0.3][r % 8] for r in range(R)], device=DEV)
    keys = torch.tensor([noise_key(5, r, 1000 + 17 * r) for r in range(R)], dtype=torch.int64, device=DEV)
    assert _exact_draws(logits[:3, :1001], temps[:3], keys[:3]) == \
        [plain.sample(logits[r, :1001].cpu(), float(temps[r]), seed=5, request=r, position=1000 + 17 * r) for r in range(3)]
    got = k.sample(logits, temps, keys).tolist()
    assert got == _exact_draws(logits, temps, keys)


def test_sampling_over_a_vocabulary_of_several_chunks(hip):
    """A row is cut into chunks of 8192 entries for the first pass: ties across chunks, a maximum
    at a chunk's edge, rows of a wider tensor (a stride that is no multiple of four), NaN entries."""
    from nano_vllm_amd.sampling.sampler import noise_key
    k = hip[torch.float32]
    V, R = 20011, 5
    wide = _rand((R, V + 3), torch.float32, 26, 2.0)
    logits = wide[:, 1:V + 1]                                       # stride V + 3, first entry unaligned
    logits[0, 8191] = logits[0, 8192] = logits[0, 20010] = 40.0     # a tie across chunks: the lowest index
    logits[1, 16384] = 40.0                                         # first entry of the last chunk
    logits[2, V - 1] = 40.0                                         # the very last entry
    logits[3, :] = float("nan")                                     # nothing wins: index 0
    logits[4, 5] = float("nan")
    temps = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.9], device=DEV)
    keys = torch.tensor([noise_key(3, r, 7) for r in range(R)], dtype=torch.int64, device=DEV)
    got = k.sample(logits, temps, keys).tolist()
    assert got[:4] == [8191, 16384, V - 1, 0]
    row = logits[4].cpu().clone()
    row[5] = -1e30                                                  # the plain draw has no rule for NaN
    assert got[4] == plain.sample(row, 0.9, seed=3, request=4, position=7)
    aligned = logits.contiguous()
    assert k.sample(aligned, temps, keys).tolist() == got


def test_sampling_frequencies_follow_the_softmax(hip):
    from nano_vllm_amd.sampling.sampler import noise_key
    l = torch.tensor([1.0, 0.0, -1.0, 0.5, -2.0, 0.2, -0.3])
    n, T = 20000, 0.8
    logits = l.to(DEV).repeat(n, 1)
    keys = torch.tensor([noise_key(1, 0, i) for i in range(n)], dtype=torch.int64, device=DEV)
    got = hip[torch.float32].sample(logits, torch.full((n,), T, device=DEV), keys)
    counts = torch.bincount(got.long().cpu(), minlength=7).double()
    p = torch.softmax(l.double() / T, 0)
    chi2 = float(((counts - n * p) ** 2 / (n * p)).sum())
    assert chi2 < 22.5                                              # 6 degrees of freedom, 0.1 % point
