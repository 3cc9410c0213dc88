"""GPU parity: grouped w8a8 GEMM (int32 accumulators bit-exact) and its two epilogues against the oracle."""
import numpy as np
import pytest
import torch

import umdk_original_amd as cam
from umdk_original_amd import synth
from gpu_util import announce, to_np, assert_bits_equal

pytestmark = pytest.mark.gpu


def _inputs(sizes, Kd, N, seed, wrange=127):
    G = len(sizes)
    gl = torch.tensor(np.cumsum(sizes), dtype=torch.int64)
    A = int(gl[-1])
    a = synth.uniform_int8((max(A, 1), Kd), seed)
    w = synth.uniform_int8((G, Kd, N), seed + 1, -wrange, wrange)
    return a, w, gl, A


@pytest.mark.parametrize("gate_up", [False, True])
@pytest.mark.parametrize("sizes,Kd,N", [
    ([5], 128, 128),
    ([1, 0, 33, 128, 129, 0, 7], 256, 256),
    ([300, 2, 0, 64], 384, 640),
    ([17, 40], 1024, 1152),
    ([700, 5, 0, 385], 128, 384),    # several row tiles per expert, shortest K loop, ragged column block
    ([257], 2048, 128),              # three uneven tiles, long K loop that wraps around its start depth
])
def test_int32_accumulators_bit_exact(gpu, oracle, sizes, Kd, N, gate_up):
    announce("gemm int32 sizes=%s Kd=%d N=%d gate_up=%s" % (sizes, Kd, N, gate_up))
    a, w, gl, A = _inputs(sizes, Kd, N, seed=Kd + N)
    wp = cam.prepack_weight(w.to(gpu), gate_up)
    got = cam.grouped_matmul_int32(a.to(gpu), wp, gl.to(gpu))
    want = oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())
    assert_bits_equal(to_np(got)[:A], want[:A], "int32 accumulators")


def test_int32_extreme_operands(gpu, oracle):
    announce("gemm int32 extremes")
    Kd, N = 7168, 128
    a = torch.full((3, Kd), -128, dtype=torch.int8)
    a[1] = 127
    a[2, ::2] = 127
    w = torch.full((1, Kd, N), -128, dtype=torch.int8)
    w[0, :, ::3] = 127
    gl = torch.tensor([3], dtype=torch.int64)
    got = cam.grouped_matmul_int32(a.to(gpu), cam.prepack_weight(w.to(gpu), False), gl.to(gpu))
    want = oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())
    assert_bits_equal(to_np(got), want, "int32 accumulators")
    assert int(got.max()) == Kd * 128 * 128


def test_group_list_as_counts_and_per_expert_tensors(gpu, oracle):
    announce("gemm counts + tensor list")
    sizes = [9, 0, 140, 3]
    a, w, gl, A = _inputs(sizes, 256, 128, seed=21)
    want = oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())
    counts = torch.tensor(sizes, dtype=torch.int64)
    wp = cam.prepack_weight(w.to(gpu), False)
    got = cam.grouped_matmul_int32(a.to(gpu), wp, counts.to(gpu), group_list_type=1)
    assert_bits_equal(to_np(got)[:A], want[:A], "counts form")
    per = [cam.prepack_weight(w[g].to(gpu), False) for g in range(len(sizes))]
    got = cam.grouped_matmul_int32(a.to(gpu), per, gl.to(gpu))
    assert_bits_equal(to_np(got)[:A], want[:A], "tensor list form")


@pytest.mark.parametrize("sizes,H,I", [([4, 0, 131, 60], 256, 128), ([128, 1, 77], 1024, 512), ([3, 200], 512, 1536)])
def test_gmm1_swiglu_quant_bit_exact(gpu, oracle, sizes, H, I):
    announce("gmm1 sizes=%s H=%d I=%d" % (sizes, H, I))
    a, w, gl, A = _inputs(sizes, H, 2 * I, seed=H + I, wrange=16)
    G = len(sizes)
    ws = synth.channel_scales((G, 2 * I), seed=31)
    xs = synth.channel_scales((max(A, 1),), seed=32, lo=0.005, hi=0.05)
    a[min(5, A - 1)] = 0  # an all-zero activation row -> all-zero product row
    y, ysc = cam.grouped_matmul_swiglu_quant(a.to(gpu), xs.to(gpu), cam.prepack_weight(w.to(gpu), True), ws.to(gpu),
                                             gl.to(gpu))
    c = oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())
    d = oracle.gmm1_epilogue(c, ws.numpy(), xs.numpy(), gl.numpy())
    want_q, want_s = oracle.swiglu_quant(d, rows=A)
    assert_bits_equal(to_np(ysc)[:A].view(np.uint32), want_s[:A].view(np.uint32), "y_scale")
    assert_bits_equal(to_np(y)[:A], want_q[:A], "y int8")
    assert (to_np(y)[min(5, A - 1)] == 0).all() and float(ysc[min(5, A - 1)]) == 0.0


@pytest.mark.parametrize("sizes,I,H", [([4, 0, 131, 60], 128, 256), ([128, 1, 77], 512, 1024), ([3, 200], 2048, 7168)])
def test_gmm2_dequant_bit_exact(gpu, oracle, sizes, I, H):
    announce("gmm2 sizes=%s I=%d H=%d" % (sizes, I, H))
    a, w, gl, A = _inputs(sizes, I, H, seed=I + H, wrange=16)
    G = len(sizes)
    ws = synth.channel_scales((G, H), seed=33)
    xs = synth.channel_scales((max(A, 1),), seed=34, lo=0.001, hi=0.01)
    out = cam.grouped_matmul_dequant(a.to(gpu), xs.to(gpu), cam.prepack_weight(w.to(gpu), False), ws.to(gpu), gl.to(gpu))
    c = oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())
    want = oracle.gmm2_epilogue(c, ws.numpy(), xs.numpy(), gl.numpy())
    assert out.dtype == torch.bfloat16
    assert_bits_equal(to_np(out)[:A], want[:A], "bf16 output")


@pytest.mark.parametrize("sizes,I,H", [([4, 0, 131, 60], 128, 256), ([300, 77], 512, 1024)])
def test_gmm2_wire_rows_bit_exact(gpu, oracle, sizes, I, H):
    """GroupedMatmulDequant with an int8 output: the bf16 rows quantised for the wire in 8-column blocks."""
    announce("gmm2 wire rows sizes=%s I=%d H=%d" % (sizes, I, H))
    a, w, gl, A = _inputs(sizes, I, H, seed=I + H + 1, wrange=16)
    G = len(sizes)
    ws = synth.channel_scales((G, H), seed=35)
    xs = synth.channel_scales((max(A, 1),), seed=36, lo=0.001, hi=0.01)
    wp = cam.prepack_weight(w.to(gpu), False)
    packed = cam.grouped_matmul_dequant(a.to(gpu), xs.to(gpu), wp, ws.to(gpu), gl.to(gpu), wire_rows=True)
    assert packed.dtype == torch.int8 and packed.shape == (max(A, 1), H + H // 4)
    c = oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())
    rows = oracle.gmm2_epilogue(c, ws.numpy(), xs.numpy(), gl.numpy())
    want = oracle.comm_quant_rows(rows[:A])
    assert np.array_equal(packed.cpu().numpy().view(np.uint8)[:A], want), "wire rows"


def test_full_size_grouped_gemm_sampled_rows(gpu):
    """One GPU's 32 local experts at the benchmark shape; sampled rows against an exact CPU integer matmul."""
    announce("gemm C3 full size, sampled rows")
    G, H, I, rows = 32, 7168, 2048, 8192
    sizes = synth.zipf_group_sizes(G, rows, seed=45)
    assert int((sizes == 0).sum()) >= 3
    gl = torch.cumsum(sizes, 0)
    a = synth.uniform_int8((rows, H), 45)
    g_cpu = torch.Generator().manual_seed(451)
    w1 = torch.randint(-127, 128, (G, H, 2 * I), generator=g_cpu, dtype=torch.int8)
    wp = cam.prepack_weight(w1.to(gpu), True)
    got = cam.grouped_matmul_int32(a.to(gpu), wp, gl.to(gpu))
    starts = (gl - sizes).tolist()
    checked = 0
    for g in range(G):
        n = int(sizes[g])
        if n == 0:
            continue
        pick = sorted({0, n - 1, n // 2})
        r = torch.tensor([starts[g] + p for p in pick])
        want = a[r].to(torch.int32) @ w1[g].to(torch.int32)  # exact
        assert torch.equal(got[r.to(gpu)].cpu(), want), "expert %d" % g
        checked += len(pick)
    assert checked >= 29
    # linearity in the activations: doubling a (within int8 range) doubles every accumulator
    a_small = torch.clamp(a, -60, 60)
    c1 = cam.grouped_matmul_int32(a_small.to(gpu), wp, gl.to(gpu))
    c2 = cam.grouped_matmul_int32((a_small * 2).to(gpu), wp, gl.to(gpu))
    assert torch.equal(c2, c1 * 2)


def _sample_rows(n):
    """Rows of an expert with n rows: both ends, the middle, the neighbours of every multiple of 32 that is also a
    multiple of 128 or 256 (tile edges of any tiling in those units), and a sparse stride through the rest."""
    pick = {0, n - 1, n // 2}
    for edge in range(0, n, 128):
        pick.update({edge - 1, edge, edge + 1, edge + 31, edge + 32, edge + 33})
    pick.update(range(5, n, 61))
    return sorted(p for p in pick if 0 <= p < n)


def test_full_size_epilogues_sampled_rows(gpu, oracle):
    """Both GEMM operators with their epilogues at the benchmark shape (32 experts, 8192 Zipf rows, H 7168,
    I 2048): y int8, y_scale and the bf16 output of sampled rows against the oracle run on exactly those rows
    (rows are independent, so a group list over the sampled rows gives bit-identical expectations)."""
    announce("gemm C3 full size, both epilogues, sampled rows")
    G, H, I, rows = 32, 7168, 2048, 8192
    sizes = synth.zipf_group_sizes(G, rows, seed=45)
    gl = torch.cumsum(sizes, 0)
    starts = (gl - sizes).tolist()
    a = synth.uniform_int8((rows, H), 45)
    a[starts[int(torch.argmax(sizes))] + 7] = 0  # an all-zero row inside the largest expert
    xs = synth.channel_scales((rows,), 451, 0.005, 0.05)
    g_cpu = torch.Generator().manual_seed(452)
    w1 = torch.randint(-127, 128, (G, H, 2 * I), generator=g_cpu, dtype=torch.int8)
    w2 = torch.randint(-127, 128, (G, I, H), generator=g_cpu, dtype=torch.int8)
    w1s = synth.channel_scales((G, 2 * I), 453)
    w2s = synth.channel_scales((G, H), 454)
    w1p = cam.prepack_weight(w1.to(gpu), True)
    w2p = cam.prepack_weight(w2.to(gpu), False)
    y, ysc = cam.grouped_matmul_swiglu_quant(a.to(gpu), xs.to(gpu), w1p, w1s.to(gpu), gl.to(gpu))
    out = cam.grouped_matmul_dequant(y, ysc, w2p, w2s.to(gpu), gl.to(gpu))
    y_c, ysc_c, out_c = y.cpu(), ysc.cpu(), out.cpu()
    checked = 0
    for g in range(G):
        n = int(sizes[g])
        if n == 0:
            continue
        r = torch.tensor([starts[g] + p for p in _sample_rows(n)])
        sub_gl = np.array([len(r)], np.int64)
        # exact integer products through float64 (|sum| <= 7168 * 127 * 127 < 2^53)
        c1 = (a[r].double() @ w1[g].double()).to(torch.int32).numpy()
        d = oracle.gmm1_epilogue(c1, w1s[g:g + 1].numpy(), xs[r].numpy(), sub_gl)
        want_q, want_s = oracle.swiglu_quant(d)
        assert_bits_equal(to_np(ysc_c[r]).view(np.uint32), want_s.view(np.uint32), "y_scale, expert %d" % g)
        assert_bits_equal(to_np(y_c[r]), want_q, "y int8, expert %d" % g)
        c2 = (y_c[r].double() @ w2[g].double()).to(torch.int32).numpy()
        want_o = oracle.gmm2_epilogue(c2, w2s[g:g + 1].numpy(), ysc_c[r].numpy(), sub_gl)
        assert_bits_equal(to_np(out_c[r]), want_o, "bf16 output, expert %d" % g)
        checked += len(r)
    assert checked >= 400
    zr = starts[int(torch.argmax(sizes))] + 7
    assert (y_c[zr] == 0).all() and float(ysc_c[zr]) == 0.0 and (out_c[zr].float() == 0).all()


def test_many_tiles_per_expert_epilogues(gpu, oracle):
    """Experts of 5 and 9 row tiles of 128 (and a ragged one) through both epilogues, every row checked."""
    announce("gemm epilogues, many tiles per expert")
    sizes, H, I = [600, 0, 1100, 77], 512, 256
    a, w, gl, A = _inputs(sizes, H, 2 * I, seed=99, wrange=16)
    G = len(sizes)
    ws = synth.channel_scales((G, 2 * I), seed=41)
    xs = synth.channel_scales((A,), seed=42, lo=0.005, hi=0.05)
    y, ysc = cam.grouped_matmul_swiglu_quant(a.to(gpu), xs.to(gpu), cam.prepack_weight(w.to(gpu), True), ws.to(gpu),
                                             gl.to(gpu))
    c = oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())
    want_q, want_s = oracle.swiglu_quant(oracle.gmm1_epilogue(c, ws.numpy(), xs.numpy(), gl.numpy()), rows=A)
    assert_bits_equal(to_np(ysc).view(np.uint32), want_s.view(np.uint32), "y_scale")
    assert_bits_equal(to_np(y), want_q, "y int8")
    w2 = synth.uniform_int8((G, I, H), 98, -16, 16)
    w2s = synth.channel_scales((G, H), seed=43)
    out = cam.grouped_matmul_dequant(y, ysc, cam.prepack_weight(w2.to(gpu), False), w2s.to(gpu), gl.to(gpu))
    c2 = oracle.gmm_int32(want_q, w2.numpy(), gl.numpy())
    want = oracle.gmm2_epilogue(c2, w2s.numpy(), want_s, gl.numpy())
    assert_bits_equal(to_np(out), want, "bf16 output")


def test_gmm2_fp16_output_bit_exact(gpu, oracle):
    """GroupedMatmulDequant writing IEEE fp16 (the layer's activation type when the tokens are fp16)."""
    announce("gmm2 fp16 output")
    sizes, I, H = [140, 0, 33], 512, 1024
    a, w, gl, A = _inputs(sizes, I, H, seed=91, wrange=16)
    ws = synth.channel_scales((len(sizes), H), seed=92)
    xs = synth.channel_scales((A,), seed=93, lo=0.001, hi=0.01)
    out = cam.grouped_matmul_dequant(a.to(gpu), xs.to(gpu), cam.prepack_weight(w.to(gpu), False), ws.to(gpu), gl.to(gpu),
                                     out_dtype=torch.float16)
    c = oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())
    want = oracle.gmm2_epilogue_act(c, ws.numpy(), xs.numpy(), gl.numpy(), True)
    assert out.dtype == torch.float16
    assert_bits_equal(out.cpu().view(torch.int16).numpy().view(np.uint16)[:A], want[:A], "fp16 output")


@pytest.mark.parametrize("Kd,N,gate_up", [(256, 1024, False), (192 + 64, 1280, True), (128, 576, False)])
def test_many_flat_items_per_workgroup_bit_exact(gpu, oracle, Kd, N, gate_up):
    """A decode-like group list: 300 experts of 0-9 rows, i.e. 600-900 flat items on 256 workgroups, so that every
    workgroup runs several flat items one after the other (the successor is taken and its first stages are
    touched between the K loop and the epilogue; short K loops end without requesting stages), with ragged
    column blocks and empty experts in between."""
    announce("gemm many flat items Kd=%d N=%d gate_up=%s" % (Kd, N, gate_up))
    rng = np.random.default_rng(Kd + N)
    sizes = [int(v) for v in rng.integers(0, 10, size=300)]
    a, w, gl, A = _inputs(sizes, Kd, N, seed=Kd * 3 + N)
    wp = cam.prepack_weight(w.to(gpu), gate_up)
    got = cam.grouped_matmul_int32(a.to(gpu), wp, gl.to(gpu))
    want = oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())
    assert_bits_equal(to_np(got)[:A], want[:A], "int32 accumulators")
    if not gate_up:
        G = len(sizes)
        ws = synth.channel_scales((G, N), seed=41)
        xs = synth.channel_scales((max(A, 1),), seed=42, lo=0.001, hi=0.01)
        out = cam.grouped_matmul_dequant(a.to(gpu), xs.to(gpu), wp, ws.to(gpu), gl.to(gpu))
        assert_bits_equal(to_np(out)[:A], oracle.gmm2_epilogue(want, ws.numpy(), xs.numpy(), gl.numpy())[:A], "bf16 output")


def test_long_schedule_shared_queues_bit_exact(gpu, oracle):
    """A schedule of more than twelve items per workgroup (tall experts of 2-6 row tiles with flat and empty ones
    in between): the builder then deals the items to one shared queue per XCD, flat items spread among the tall
    ones, and every workgroup asks for every item.  Every accumulator is checked."""
    rng = np.random.default_rng(77)
    sizes = []
    for _ in range(120):
        sizes.append(int(rng.integers(300, 1500)))
        if rng.random() < 0.3:
            sizes.append(int(rng.integers(0, 129)))
    Kd, N = 128, 2048
    items = sum(((s + 255) // 256) * (N // 256) if s > 128 else ((N + 511) // 512 if s > 0 else 0) for s in sizes)
    cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    announce("gemm long schedule: %d experts, %d rows, %d items on %d workgroups" % (len(sizes), sum(sizes), items, cus))
    if items < 12 * cus:
        pytest.skip("this device has too many CUs for the shape to reach the shared-queue form")
    a, w, gl, A = _inputs(sizes, Kd, N, seed=177)
    wp = cam.prepack_weight(w.to(gpu), False)
    got = cam.grouped_matmul_int32(a.to(gpu), wp, gl.to(gpu))
    want = oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())
    assert_bits_equal(to_np(got)[:A], want[:A], "int32 accumulators")


def _schedule_items(ws):
    """The tile records of the schedule a grouped-GEMM operator left at the head of its workspace."""
    from umdk_original_amd import _lib
    _, head_words, item_words, sched_at = _lib.gemm_timeline_info()
    words = ws[sched_at:sched_at + (ws.numel() - sched_at) // 4 * 4].view(torch.int32)
    n_items, n_queues, flags = int(words[0]), int(words[2]), int(words[3])
    rec = words[head_words:head_words + n_items * item_words].cpu().numpy().reshape(n_items, item_words)
    starts = words[4:4 + n_queues + 1].cpu().numpy()
    return rec, starts, n_queues, flags


@pytest.mark.parametrize("name,sizes,N", [
    ("own queues, tall and flat", [700, 5, 0, 385, 128, 129, 64, 1100], 1280),
    ("own queues, all flat", [int(v) for v in np.random.default_rng(5).integers(0, 10, size=300)], 1024),
    ("shared queues", [int(v) for v in np.random.default_rng(6).integers(250, 1300, size=160)] + [7, 0, 90, 128], 2048),
])
def test_schedule_covers_every_tile_exactly_once(gpu, name, sizes, N):
    """The device-built schedule itself: every 32-row unit of every (expert, column block) appears in exactly one
    tile, tiles respect the shape limits, and the queues partition the tile list."""
    from umdk_original_amd import _lib
    Kd = 128
    a, w, gl, A = _inputs(sizes, Kd, N, seed=11)
    wp = cam.prepack_weight(w.to(gpu), False)
    out = torch.zeros((max(A, 1), N), dtype=torch.int32, device=gpu)
    ws = _lib.call("GroupedMatmulInt32", [a.to(gpu), [wp], 0, gl.to(gpu), 0, out])
    torch.cuda.synchronize()
    rec, starts, n_queues, flags = _schedule_items(ws)
    cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    announce("schedule %s: %d tiles, %d queues, flags %d" % (name, len(rec), n_queues, flags))
    first = np.concatenate([[0], np.cumsum(sizes)[:-1]])
    nb_tall, nb_flat = (N + 255) // 256, (N + 511) // 512
    cover = {}
    for g, m0, rows, split, nb, flat, _, _ in rec.tolist():
        split, nb, flat = split & 0xffff, nb & 0xffff, flat & 0xffff  # a clock-stamping build uses the upper halves
        assert 0 <= g < len(sizes) and sizes[g] > 0
        rel = m0 - int(first[g])
        if flat:
            assert sizes[g] <= 128 and rel == 0 and rows == sizes[g] and 0 <= nb < nb_flat
            units = [(g, nb, 0)]
        else:
            assert sizes[g] > 128 and rel >= 0 and rel % 32 == 0 and 0 < rows <= 256 and rel + rows <= sizes[g]
            assert 0 <= nb < nb_tall and split == 32 * ((rows + 63) // 64)
            assert rows % 32 == 0 or rel + rows == sizes[g]
            units = [(g, nb, rel // 32 + k) for k in range((rows + 31) // 32)]
        for u in units:
            cover[u] = cover.get(u, 0) + 1
    want = {}
    for g, s in enumerate(sizes):
        if s > 128:
            for nb in range(nb_tall):
                for k in range((s + 31) // 32):
                    want[(g, nb, k)] = 1
        elif s > 0:
            for nb in range(nb_flat):
                want[(g, nb, 0)] = 1
    assert cover == want
    assert starts[0] == 0 and starts[-1] == len(rec) and (np.diff(starts) >= 0).all()
    shared = bool(flags & 2)
    assert n_queues == (8 if shared else cus)
    assert shared == (len(rec) // cus >= 12)


def test_hardware_bf16_conversion_equals_the_definition_on_all_inputs(gpu):
    """The GEMM and combine epilogues round fp32 to bf16 with the hardware's packed conversion; the oracle rounds by
    the arithmetic definition (nearest even on the bit pattern, NaN -> truncated payload with the quiet bit).  The
    calibration library compares the two over every one of the 2^32 bit patterns."""
    import ctypes
    from umdk_original_amd import build
    announce("hardware bf16 conversion against its definition, all 2^32 patterns")
    lib = ctypes.CDLL(build.CALIB_LIB_PATH)
    out = (ctypes.c_double * 4)()
    assert lib.camCalibBf16Conversion(out) == 0
    assert out[0] == 0.0, "first differing pattern 0x%08x" % int(out[1])
