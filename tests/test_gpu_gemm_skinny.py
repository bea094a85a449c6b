"""The few-token grouped matmul kernel (oxq_gemm_skinny.hpp: 16 x 16 x 32 int8 MFMA, weight rows read as contiguous
runs through a per-wave LDS strip, a group's tokens staged in LDS) through the C ABI against the CPU oracle:
integer sub-block sums bit-exact, fp32 within 1e-5 * |y_ref|_inf.  Every case asserts that the library really took
this kernel (oxq_last_launch), so a change of launch policy cannot quietly turn these into tests of the tile kernel."""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from oxillama_amd import synth
from test_gpu_parity import assert_close, canonical_ref, say

pytestmark = pytest.mark.gpu

FORMATS = [O.Q4_K, O.IQ4_XS, O.Q4_0, O.Q4_1, O.IQ4_NL]
# Q6_K, Q3_K, Q2_K (a scale per 16 weights: two MFMAs per sub-block, the integer sums per half), Q8_0 (544 bytes of a
# row per step), Q5_K, Q5_0, Q5_1: the kernel's one-token-tile shapes only; expert groups of more than 16 rows take
# further passes
ONE_TILE = [O.Q6_K, O.Q8_0, O.Q5_K, O.Q3_K, O.Q2_K, O.Q5_0, O.Q5_1]
FORMATS_1TILE = FORMATS + ONE_TILE


def weights(t, seed, n, k_):
    """Synthetic weights: the package's generator for the five formats it knows, the oracle's random blocks otherwise."""
    if t in synth.BLOCK:
        return synth.weights(t, seed, n, k_)
    return O.random_blocks(t, seed, n, k_)


def sum_groups(t, k_):
    return k_ // O.GROUP_COLS[t]


def ref_sums(ref, t, w, act_row, n, k_):
    """The integer sums the kernel's dump holds: the reference's; for Q4_0 of the unsigned nibbles (sum q a = sum (q - 8) a
    + 8 sum a: the "- 8" enters in fp32, as in the tile kernel)."""
    s = ref.block_sums(t, w, act_row, n, k_)
    if t in (O.Q4_0, O.Q5_0):  # (Q5_0: the unsigned 5-bit values, "- 16" in fp32)
        a = act_row.reshape(k_ // 32, 34)[:, 2:].view(np.int8).astype(np.int32).sum(axis=1)
        s = s + (8 if t == O.Q4_0 else 16) * a[None, :]
    return s


def shaped_rows(counts, max_rows):
    """Rows per expert the library shapes a grouped launch for: the caller's bound, or twice the mean."""
    total = sum(counts)
    if max_rows:
        return min(max_rows, total)
    return min(2 * ((total + len(counts) - 1) // len(counts)), total)


def last_launch():
    from oxillama_amd import capi
    buf = C.create_string_buffer(256)
    capi.load().oxq_last_launch(buf, 256)
    return buf.value.decode()


def _case(ref, t, counts, n, k_, seed):
    """Experts with the given token-row counts: offsets, Q8_0 activation rows, weights."""
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(offsets[-1])
    x = synth.normal_f32(seed, rows * k_).reshape(rows, k_)
    acts = ref.quantize_q8_0(x.reshape(-1)).reshape(rows, k_ // 32 * 34)
    w = np.stack([weights(t, seed + 10 + e, n, k_) for e in range(len(counts))])
    return offsets, acts, w


def _oracle_rows(ref, t, w, acts, offsets, n, k_, sample):
    y, s = {}, {}
    for r in sample:
        e = int(np.searchsorted(offsets, r, side="right") - 1)
        y[r] = canonical_ref(ref, t, w[e], acts[r], n, k_, threads=16)
        s[r] = ref_sums(ref, t, w[e], acts[r], n, k_)
    return y, s


def _run(hip, t, w, acts, offsets, n, k_, max_rows, sums=False, accumulate=False, out=None):
    import torch
    rows = int(offsets[-1])
    kern = hip.HipKernel(t)
    ws = torch.empty(kern.moe_gemm_workspace_bytes(rows, n, k_), dtype=torch.uint8, device="cuda")
    dw, da, doff = torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda(), torch.from_numpy(offsets).cuda()
    dy = out if out is not None else torch.full((rows + 2, n), 7.0, dtype=torch.float32, device="cuda")
    dsum = torch.full((rows, n, sum_groups(t, k_)), -1, dtype=torch.int32, device="cuda") if sums else None
    kern.moe_gemm_q8_dev(dw, w[0].nbytes, len(offsets) - 1, da, doff, rows, max_rows, dy, n, k_, ws,
                         accumulate=accumulate, d_sums=dsum)
    torch.cuda.synchronize()
    return dy, dsum


# (row counts per expert, n, k, max_rows handed to the call): one token tile / two (the default takes two only with
# many row groups, or enough for every compute unit once k is halved, and a mean of at most 16 rows per expert); few row groups / at least two per compute unit; an expert without rows; ragged n (a wave past the last row, a tile cut at n % 16); k of one step, of a
# whole number of chunks and with a short last chunk; groups larger than the launch is shaped for (max_rows = 0: the
# shape follows twice the mean, the largest group takes further passes over its weights)
CASES = [
    ([3, 0, 16, 1], 300, 512, 16),
    ([5, 9, 2, 16, 7, 1, 0, 11], 72, 1536, 16),
    ([16, 16], 128, 2560, 16),
    ([12, 7, 16, 3, 9, 14, 2, 5], 8192, 512, 16),
    ([20, 3, 15, 4, 17, 1, 19, 12], 8192, 1024, 20),
    ([32, 1, 17, 0, 8, 30, 2, 5], 8200, 512, 32),
    ([2, 1, 40, 1, 3, 0, 1, 2], 96, 1024, 0),
    ([9, 50, 3, 2, 1, 0, 20, 5], 8192, 512, 0),
    # two token tiles on few row groups per expert: each expert's k in two halves, the halves' sums added by a second
    # launch (one step per half; several chunks per half and groups of unknown size)
    ([20, 3, 17, 0, 32, 16, 9, 25], 2048, 1024, 32),
    ([22, 10, 17, 13, 20, 16, 9, 15], 4096, 3072, 0),
    # one token tile on few row groups per expert (Q6_K, Q8_0: k in two halves there as well)
    ([16, 5, 0, 9, 12, 1, 16, 7], 2048, 2048, 16),
    # a mean of 17 rows, sizes unknown to the host: shaped for twice that, more than two token tiles hold
    ([25, 18, 19, 16, 12, 21, 10, 15], 8192, 1024, 0),
    # an odd number of super-blocks (the last step has one live half): three, five (a chunk boundary inside), eleven
    ([3, 0, 16, 1], 300, 768, 16),
    ([12, 7, 16, 3, 9, 14, 2, 5], 8192, 1280, 16),
    ([20, 3, 15, 4, 17, 1, 19, 12], 8192, 2816, 20),
]


@pytest.mark.parametrize("t", FORMATS_1TILE, ids=lambda t: O.NAMES[t])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "r%d_n%d_k%d_max%d" % (sum(c[0]), c[1], c[2], c[3]))
def test_skinny_grouped_against_oracle(hip, ref, t, case):
    counts, n, k_, max_rows = case
    say("skinny", O.NAMES[t], case)
    # (Q6_K, Q8_0 shaped for 17..32 rows: the one-tile kernel, a second pass over the weights for the larger groups)
    offsets, acts, w = _case(ref, t, counts, n, k_, 4100 + n + k_)
    rows = int(offsets[-1])
    dy, dsum = _run(hip, t, w, acts, offsets, n, k_, max_rows, sums=True)
    assert last_launch().startswith("gemm_skinny_kernel"), last_launch()
    y, s = dy.cpu().numpy(), dsum.cpu().numpy()
    assert np.all(y[rows:] == 7.0)  # guard rows
    sample = range(rows) if n <= 512 else sorted(set(list(range(0, rows, 7)) + [int(o) for o in offsets[:-1] if o < rows] +
                                                      [int(o) - 1 for o in offsets[1:] if o > 0]))
    y_ref, s_ref = _oracle_rows(ref, t, w, acts, offsets, n, k_, sample)
    for r in sample:
        assert_close(y[r], y_ref[r], f"skinny {case} row {r}")
        assert np.array_equal(s[r], s_ref[r]), f"integer sums of row {r}"
    # the production launch (no sums): the same bits; overwrite then accumulate: twice them
    dy2, _ = _run(hip, t, w, acts, offsets, n, k_, max_rows)
    assert last_launch().startswith("gemm_skinny_kernel"), last_launch()
    import torch
    assert torch.equal(dy2, dy)
    dy3, _ = _run(hip, t, w, acts, offsets, n, k_, max_rows, accumulate=True, out=dy2.clone())
    assert torch.equal(dy3[:rows], dy[:rows] + dy[:rows]) and torch.equal(dy3[rows:], dy[rows:])


@pytest.mark.parametrize("t", [O.Q4_0, O.Q4_1, O.IQ4_NL, O.Q4_K], ids=lambda t: O.NAMES[t])
def test_skinny_grouped_larger_groups_in_the_formats_of_32_weight_blocks(hip, ref, t):
    """A mean of 32 rows per expert (sizes unknown to the host: the launch is shaped for 64, groups beyond 32 rows take a
    second pass): the formats of 32-weight blocks stay on the few-token kernel up to a mean of 48, Q4_K goes to the tile
    kernel from 20."""
    counts, n, k_ = [42, 24, 30, 29, 27, 34, 32, 38], 8192, 512
    offsets, acts, w = _case(ref, t, counts, n, k_, 5100)
    rows = int(offsets[-1])
    dy, _ = _run(hip, t, w, acts, offsets, n, k_, 0)
    took = last_launch()
    say(O.NAMES[t], took)
    assert took.startswith("gemm_skinny_kernel") == (t != O.Q4_K), took
    y = dy.cpu().numpy()
    assert np.all(y[rows:] == 7.0)
    sample = sorted(set(list(range(0, rows, 11)) + [int(o) for o in offsets[:-1]] + [int(o) - 1 for o in offsets[1:]]))
    y_ref, _ = _oracle_rows(ref, t, w, acts, offsets, n, k_, sample)
    for r in sample:
        assert_close(y[r], y_ref[r], f"row {r}")


@pytest.mark.parametrize("t", FORMATS, ids=lambda t: O.NAMES[t])
def test_skinny_shapes_give_the_same_bits(hip, ref, tuning, t):
    """Every launch shape of the kernel (waves per work group, super-blocks per chunk) adds a result's terms in the same
    order; the tile kernel (another order) agrees within the fp32 bar."""
    import torch
    counts, n, k_ = [20, 3, 16, 0, 31, 9], 400, 3584
    offsets, acts, w = _case(ref, t, counts, n, k_, 977)
    rows = int(offsets[-1])
    outs = {}
    for variant in (0, 200, 201, 203, 204, 205, 99):
        tuning("gemm_variant", variant)
        dy, _ = _run(hip, t, w, acts, offsets, n, k_, 31)
        say(" variant", variant, last_launch())
        assert last_launch().startswith("gemm_tile_kernel" if variant in (0, 99) else "gemm_skinny_kernel"), last_launch()
        outs[variant] = dy[:rows].clone()
    for variant in (201, 203, 204, 205):
        assert torch.equal(outs[variant], outs[200]), variant
    assert torch.equal(outs[0], outs[99])  # two token tiles on few row groups: the default is the tile kernel
    assert_close(outs[200].cpu().numpy(), outs[99].cpu().numpy(), "skinny against tile kernel")


@pytest.mark.parametrize("t", FORMATS_1TILE, ids=lambda t: O.NAMES[t])
@pytest.mark.parametrize("m", [1, 16, 17, 32])
def test_skinny_plain_matmul_forced(hip, ref, tuning, t, m):
    """One matrix, no experts (the default there is the tile kernel; the kernel is selectable), ragged n."""
    import torch
    if t in ONE_TILE and m > 16:
        pytest.skip("two token tiles: the tile kernel's case for this format")
    n, k_ = 1000, 2048
    w = weights(t, 31, n, k_)
    x = synth.normal_f32(32 + m, m * k_)
    acts = ref.quantize_q8_0(x).reshape(m, k_ // 32 * 34)
    kern = hip.HipKernel(t)
    tuning("gemm_tile_min_rows", 1)
    tuning("gemm_variant", 200 if t in ONE_TILE else 204)
    ws = torch.empty(kern.gemm_workspace_bytes(m, n, k_), dtype=torch.uint8, device="cuda")
    dy = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    kern.gemm_q8_dev(torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda(), dy, m, n, k_, workspace=ws)
    torch.cuda.synchronize()
    assert last_launch().startswith("gemm_skinny_kernel"), last_launch()
    y = dy.cpu().numpy()
    for r in range(m):
        assert_close(y[r], canonical_ref(ref, t, w, acts[r], n, k_), f"plain m={m} row {r}")


def test_skinny_full_size_c5_gate(hip, ref):
    """C5's gate shape, 8 experts of IQ4_XS 14336 x 4096, up to 16 rows each and up to 32: oracle on sampled rows."""
    t, n, k_ = O.IQ4_XS, 14336, 4096
    for counts in ([11, 11, 9, 6, 10, 3, 9, 5], [20, 3, 15, 4, 17, 1, 19, 12]):
        offsets, acts, w = _case(ref, t, counts, n, k_, 6000 + counts[0])
        rows = int(offsets[-1])
        dy, _ = _run(hip, t, w, acts, offsets, n, k_, max(counts))
        assert last_launch().startswith("gemm_skinny_kernel"), last_launch()
        y = dy.cpu().numpy()
        for r in list(range(0, rows, 13)) + [rows - 1]:
            e = int(np.searchsorted(offsets, r, side="right") - 1)
            assert_close(y[r], canonical_ref(ref, t, w[e], acts[r], n, k_, threads=16), f"c5 gate row {r} expert {e}")
        del dy


@pytest.mark.parametrize("t", FORMATS_1TILE, ids=lambda t: O.NAMES[t])
@pytest.mark.parametrize("shape", [(16, 4096, 8192), (9, 8200, 4096), (6, 16384, 2048), (13, 2100, 16384), (11, 16384, 3584), (7, 8201, 4096),
                                   # 17..32 rows on fewer than 8192 weight rows: two token tiles (Q6_K, Q8_0: two passes)
                                   (21, 4096, 8192), (32, 2100, 16384), (17, 4100, 8192),
                                   # an odd number of super-blocks (43, 17): the last split ends on half a step
                                   (16, 4096, 11008), (9, 8200, 4352), (21, 4096, 11008)],
                         ids=lambda s: "x".join(map(str, s)))
def test_skinny_one_matrix_split_k(hip, ref, t, shape):
    """One matrix, up to 16 token rows (32 on fewer than 8192 weight rows), at least 2^25 weights: k is split over work groups, each writes its sums for its
    part of k, a second launch adds the parts in index order.  Integer sums ==, fp32 1e-5, bias, accumulate, ragged n,
    splits of unequal length."""
    import torch
    from oxillama_amd import linear
    m, n, k_ = shape
    say("skinny split-k", O.NAMES[t], shape)
    w = weights(t, 71, n, k_)
    acts = ref.quantize_q8_0(synth.normal_f32(72 + m, m * k_)).reshape(m, k_ // 32 * 34)
    bias = synth.normal_f32(73, n)
    kern = hip.HipKernel(t)
    dw, da, db = torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda(), torch.from_numpy(bias).cuda()
    ws = torch.empty(kern.gemm_workspace_bytes(m, n, k_), dtype=torch.uint8, device="cuda")
    dy = torch.full((m + 1, n), 7.0, dtype=torch.float32, device="cuda")
    dsum = torch.full((m, n, sum_groups(t, k_)), -1, dtype=torch.int32, device="cuda")
    kern.gemm_block_sums_dev(dw, da, dy, dsum, m, n, k_, workspace=ws)
    torch.cuda.synchronize()
    assert last_launch().startswith("gemm_skinny_kernel"), last_launch()
    y, s = dy.cpu().numpy(), dsum.cpu().numpy()
    assert np.all(y[m:] == 7.0)
    rows = sorted(set([0, m - 1, m // 2]))
    y_ref = {r: canonical_ref(ref, t, w, acts[r], n, k_, threads=16) for r in rows}
    for r in rows:
        assert_close(y[r], y_ref[r], f"split-k {shape} row {r}")
        assert np.array_equal(s[r], ref_sums(ref, t, w, acts[r], n, k_)), f"integer sums of row {r}"
    # production launch: the same bits; accumulate: twice them; bias in the reduction
    dy2 = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    kern.gemm_q8_dev(dw, da, dy2, m, n, k_, workspace=ws)
    assert last_launch().startswith("gemm_skinny_kernel"), last_launch()
    kern.gemm_q8_dev(dw, da, dy2, m, n, k_, accumulate=True, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(dy2, dy[:m] + dy[:m])
    dy3 = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    linear.linear_forward_batch_dev(t, dw, da, dy3, m, n, k_, d_bias=db, workspace=ws)
    torch.cuda.synchronize()
    assert last_launch().startswith("gemm_skinny_kernel"), last_launch()
    assert torch.equal(dy3, dy[:m] + db[None, :])
    # a workspace of the re-tiled activations' size alone, without room for the per-split sums, is refused
    from oxillama_amd import capi
    planes = ((k_ // 32) * (((m + 127) // 128) * 128 + 128) * 46 + 255) // 256 * 256
    dy4 = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    small = ws[:planes]
    st = capi.load().oxq_gemm_q8_dev(t, dw.data_ptr(), da.data_ptr(), dy4.data_ptr(), m, n, k_, 0, small.data_ptr(),
                                     small.numel(), None)
    assert st == capi.ERR_BUFFER_TOO_SMALL


def test_skinny_one_matrix_with_many_row_groups(hip, ref):
    """One matrix with at least two groups of 128 rows per compute unit (a vocabulary projection) and up to 16 token
    rows: the few-token kernel without a split of k."""
    import torch
    t, m, n, k_ = O.Q4_K, 9, 65600, 512
    w = synth.weights(t, 85, n, k_)
    acts = ref.quantize_q8_0(synth.normal_f32(86, m * k_)).reshape(m, k_ // 32 * 34)
    kern = hip.HipKernel(t)
    ws = torch.empty(kern.gemm_workspace_bytes(m, n, k_), dtype=torch.uint8, device="cuda")
    dy = torch.full((m + 1, n), 7.0, dtype=torch.float32, device="cuda")
    dsum = torch.full((m, n, k_ // 32), -1, dtype=torch.int32, device="cuda")
    kern.gemm_block_sums_dev(torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda(), dy, dsum, m, n, k_, workspace=ws)
    torch.cuda.synchronize()
    assert last_launch().startswith("gemm_skinny_kernel"), last_launch()
    y, s = dy.cpu().numpy(), dsum.cpu().numpy()
    assert np.all(y[m:] == 7.0)
    for r in (0, 4, m - 1):
        assert_close(y[r], canonical_ref(ref, t, w, acts[r], n, k_, threads=16), f"many row groups, row {r}")
        assert np.array_equal(s[r], ref.block_sums(t, w, acts[r], n, k_))


def test_skinny_split_k_on_the_host_routes(hip, ref):
    """The routes that size their own scratch -- QuantKernel::gemm on host slices, oxq_gemm_q8_dev without a
    workspace -- leave room for the per-split sums and take the same kernel."""
    import torch
    t, m, n, k_ = O.Q4_K, 8, 8192, 4096
    w = weights(t, 81, n, k_)
    x = synth.normal_f32(82, m * k_)
    acts = ref.quantize_q8_0(x).reshape(m, k_ // 32 * 34)
    kern = hip.HipKernel(t)
    y = np.zeros(m * n, dtype=np.float32)
    kern.gemm(hip.QuantTensor(w, [n, k_], t), x, y, m, n, k_)
    assert last_launch().startswith("gemm_skinny_kernel"), last_launch()
    y = y.reshape(m, n)
    for r in (0, 3, m - 1):
        assert_close(y[r], canonical_ref(ref, t, w, acts[r], n, k_, threads=16), f"host gemm row {r}")
    dy = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    kern.gemm_q8_dev(torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda(), dy, m, n, k_)  # library-owned scratch
    torch.cuda.synchronize()
    assert last_launch().startswith("gemm_skinny_kernel"), last_launch()
    assert np.array_equal(dy.cpu().numpy(), y)


@pytest.mark.parametrize("case", [(O.IQ4_XS, 3, 8192, 4096), (O.Q4_K, 5, 4096, 8192), (O.Q4_K, 4, 8192, 4096),
                                  (O.Q6_K, 5, 4096, 8192), (O.Q6_K, 4, 4096, 8192)],
                         ids=lambda c: "%s_m%d_%dx%d" % (O.NAMES[c[0]], c[1], c[2], c[3]))
def test_few_rows_take_the_few_token_kernel_when_a_workspace_has_room(hip, ref, case):
    """Below the tile kernel's row threshold the GEMV launches serve a matmul, four rows per pass -- except where the
    few-token kernel is faster still (from 3 rows where a GEMV launch takes two vectors at most, else from 5, on shapes it splits over k) and the caller's
    workspace has room for its sums.  Without a workspace, or with a small one, the GEMV launches stay."""
    import torch
    t, m, n, k_ = case
    w = synth.weights(t, 91, n, k_)
    acts = ref.quantize_q8_0(synth.normal_f32(92, m * k_)).reshape(m, k_ // 32 * 34)
    kern = hip.HipKernel(t)
    dw, da = torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda()
    ws = torch.empty(kern.gemm_workspace_bytes(m, n, k_), dtype=torch.uint8, device="cuda")
    # from 3 rows where a GEMV launch takes at most two vectors (rows of 2 or 5..8 steps of 64 lanes), else from 5
    steps = -(-(k_ // (32 if t == O.IQ4_XS else 64)) // 64)
    expect_skinny = m >= (5 if steps in (1, 3, 4) else 3)
    outs = []
    for workspace in (ws, ws[:4096], None):
        dy = torch.zeros((m, n), dtype=torch.float32, device="cuda")
        kern.gemm_q8_dev(dw, da, dy, m, n, k_, workspace=workspace)
        torch.cuda.synchronize()
        took = last_launch()
        say(" ", O.NAMES[t], m, "workspace", None if workspace is None else workspace.numel(), "->", took)
        assert took.startswith("gemm_skinny_kernel") == (expect_skinny and workspace is ws), took
        outs.append(dy.cpu().numpy())
    for r in range(m):
        y_ref = canonical_ref(ref, t, w, acts[r], n, k_, threads=16)
        for y in outs:
            assert_close(y[r], y_ref, f"few rows {case} row {r}")


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
@pytest.mark.parametrize("counts", [[1, 0, 0, 1, 0, 0, 0, 0], [2, 0, 1, 0, 0, 3, 0, 2], [0, 0, 8]], ids=lambda c: "r%d" % sum(c))
def test_grouped_matmul_of_a_handful_of_rows_is_one_gemv_launch(hip, ref, t, counts):
    """Up to 8 token rows in all (a single token's top-2, a decode batch of a few): one GEMV launch, a matvec per row
    against its expert's matrix -- the bits of oxq_matvec_q8_fused_dev on that row, for every format."""
    import torch
    n, k_ = 300, 2048
    offsets, acts, w = _case(ref, t, counts, n, k_, 7000 + sum(counts))
    rows = int(offsets[-1])
    dy, _ = _run(hip, t, w, acts, offsets, n, k_, max(counts))
    assert last_launch().startswith("gemv_q8_cached"), last_launch()
    y = dy.cpu().numpy()
    assert np.all(y[rows:] == 7.0)
    kern = hip.HipKernel(t)
    for r in range(rows):
        e = int(np.searchsorted(offsets, r, side="right") - 1)
        assert_close(y[r], canonical_ref(ref, t, w[e], acts[r], n, k_), f"row {r} expert {e}")
        d1 = torch.zeros(n, dtype=torch.float32, device="cuda")
        kern.matvec_q8_fused_dev(torch.from_numpy(w[e]).cuda(), torch.from_numpy(acts[r]).cuda(), d1, n, k_, accumulate=False)
        torch.cuda.synchronize()
        assert np.array_equal(d1.cpu().numpy(), y[r]), f"row {r}: not the single matvec's bits"
    # accumulate
    dy2, _ = _run(hip, t, w, acts, offsets, n, k_, max(counts), accumulate=True, out=dy.clone())
    assert torch.equal(dy2[:rows], dy[:rows] + dy[:rows]) and torch.equal(dy2[rows:], dy[rows:])
