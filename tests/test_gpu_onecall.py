"""Small batches (at most 512 segments and 1024 segment-head pairs) through ba_gemm_softmax_static: ONE launch that reads the metadata
itself -- no scheduler launch, no plan.  Every segment class against the oracle, the prefix sums it writes
bit for bit, rejected metadata, caller-given prefix sums with gaps, and replays from a HIP graph."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from blockedattention_amd import capi
from _util import assert_probs_close, dev_i64, make_plan, random_operands

pytestmark = pytest.mark.gpu


def mixed_batch(rng, nseg):
    """Every class of segment: strips of all widths, tiny ones, tile-class, leftovers, unaligned, empty, K = 0."""
    M = rng.integers(1, 120, nseg); N = rng.integers(1, 257, nseg); K = rng.choice(np.arange(8, 129, 8), nseg)
    special = [(150, 700, 128), (40, 300, 64), (70, 200, 256), (33, 1, 64), (20, 50, 200), (0, 55, 64), (44, 0, 64),
               (40, 300, 0), (25, 60, 0), (5, 7, 16), (6, 8, 16), (300, 64, 128)]
    for i, (m, n, k) in enumerate(special[:max(0, nseg - 3)]):
        M[i + 1], N[i + 1], K[i + 1] = m, n, k
    if nseg >= 4:       # K not a multiple of 8 (element-wise path); areas in whole 16-byte units, so that the heads stay aligned
        M[-2], N[-2], K[-2] = 10, 40, 12
        M[-1], N[-1], K[-1] = 16, 32, 7
    return M.astype(np.int64), N.astype(np.int64), K.astype(np.int64)


def run_static(dev, M, N, K, H, dtype, scale, seed, out_dtype=None):
    A, B = random_operands(M, N, K, H, dtype, seed)
    d1, d2, do = int((M * K).sum()), int((N * K).sum()), int((M * N).sum())
    acc = [torch.full((len(M) + 1,), -7, dtype=torch.int64, device=dev) for _ in range(3)]
    out = torch.full((H, do), float("nan"), dtype=out_dtype or dtype, device=dev)
    capi.gemm_softmax_static(dev_i64(M, dev), dev_i64(N, dev), dev_i64(K, dev), A.to(dev), B.to(dev), out, H, d1, d2, do,
                             scale, *acc)
    torch.cuda.synchronize()
    for got, ref in zip(acc, oracle.lists_to_accum(M, N, K)):
        assert np.array_equal(got.cpu().numpy(), ref), "prefix sums differ from the oracle's"
    assert_probs_close(out, oracle.per_segment_torch(A, B, M, N, K, scale), f"one launch, {len(M)} segments")
    return A, B, out


@pytest.mark.parametrize("nseg", [1, 15, 64, 65, 200, 256, 257, 512])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_every_class_of_segment(dev, nseg, dtype):
    rng = np.random.default_rng(100 + nseg)
    M, N, K = mixed_batch(rng, nseg)
    run_static(dev, M, N, K, 3 if nseg <= 65 else 2, dtype, 0.17, seed=nseg)


def test_fp32_probabilities_and_one_head(dev):
    rng = np.random.default_rng(7)
    M, N, K = mixed_batch(rng, 40)
    run_static(dev, M, N, K, 1, torch.bfloat16, 0.09, seed=3, out_dtype=torch.float32)


def test_same_bits_as_the_plan_driven_call_where_no_segments_are_packed(dev):
    rng = np.random.default_rng(11)
    n = 90
    M = rng.integers(17, 200, n).astype(np.int64); N = rng.integers(17, 257, n).astype(np.int64)
    K = rng.choice(np.arange(16, 129, 16), n).astype(np.int64)
    N[3], M[3], K[3] = 520, 140, 136      # a large segment that both calls run through the tile kernel's body
    H, dtype, scale = 2, torch.float16, 0.125
    A, B, got = run_static(dev, M, N, K, H, dtype, scale, seed=5)
    plan = make_plan(dev, M, N, K, read=False)
    d1, d2, do = int((M * K).sum()), int((N * K).sum()), int((M * N).sum())
    want = torch.full((H, do), float("nan"), dtype=dtype, device=dev)
    capi.gemm_softmax(plan, A.to(dev), B.to(dev), want, H, d1, d2, do, scale)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_rejected_metadata_leaves_the_output_alone(dev):
    M = np.array([20, 30, 40], np.int64); N = np.array([24, 36, 48], np.int64); K = np.array([32, 32, 32], np.int64)
    A, B = random_operands(M, N, K, 1, torch.float16, 1)
    d1, d2, do = int((M * K).sum()), int((N * K).sum()), int((M * N).sum())
    out = torch.full((1, do), float("nan"), dtype=torch.float16, device=dev)
    Ad, Bd = A.to(dev), B.to(dev)
    bad_M = M.copy(); bad_M[1] = -3
    capi.gemm_softmax_static(dev_i64(bad_M, dev), dev_i64(N, dev), dev_i64(K, dev), Ad, Bd, out, 1, d1, d2, do, 1.0)
    torch.cuda.synchronize()
    assert torch.isnan(out).all(), "a negative size must stop the whole call"
    info, st = capi.static_read(raise_on_bad=False)
    assert st == 5 and info.bad_segments == 1 and info.nseg == 3, (st, info.bad_segments, info.nseg)
    capi.gemm_softmax_static(dev_i64(M, dev), dev_i64(N, dev), dev_i64(K, dev), Ad, Bd, out, 1, d1, d2, do + 8, 1.0)
    torch.cuda.synchronize()
    assert torch.isnan(out).all(), "totals that do not match the tensors' sizes must stop the whole call"
    info, st = capi.static_read(raise_on_bad=False)
    assert st == 5 and info.bad_segments == 0 and info.run_errors >= 1, (st, info.bad_segments, info.run_errors)
    capi.gemm_softmax_static(dev_i64(M, dev), dev_i64(N, dev), dev_i64(K, dev), Ad, Bd, out, 1, d1, d2, do, 1.0)
    torch.cuda.synchronize()
    assert_probs_close(out, oracle.per_segment_torch(A, B, M, N, K, 1.0), "after the rejected calls")
    info, st = capi.static_read()
    assert st == 0 and info.bad_segments == 0 and info.run_errors == 0 and info.Dout == do


def test_prefix_sums_given_by_the_caller_with_gaps(dev):
    rng = np.random.default_rng(21)
    n = 70
    M = rng.integers(1, 100, n).astype(np.int64); N = rng.integers(1, 200, n).astype(np.int64)
    K = rng.choice(np.arange(8, 129, 8), n).astype(np.int64)
    gap = rng.integers(0, 3, n).astype(np.int64) * 8            # holes between the segments, all three tensors
    def gapped(area):
        start = np.zeros(n + 1, np.int64)
        start[1:] = np.cumsum(area + gap)
        return start
    a1, a2, ao = gapped(M * K), gapped(N * K), gapped(M * N)
    H, dtype, scale = 2, torch.float16, 0.2
    g = torch.Generator(device="cpu").manual_seed(9)
    A = torch.randn((H, int(a1[-1])), generator=g).to(dtype); B = torch.randn((H, int(a2[-1])), generator=g).to(dtype)
    out = torch.full((H, int(ao[-1])), float("nan"), dtype=dtype, device=dev)
    capi.gemm_softmax_static(dev_i64(M, dev), dev_i64(N, dev), dev_i64(K, dev), A.to(dev), B.to(dev), out, H, int(a1[-1]),
                             int(a2[-1]), int(ao[-1]), scale, dev_i64(a1, dev), dev_i64(a2, dev), dev_i64(ao, dev),
                             mode=capi.META_GIVEN)
    torch.cuda.synchronize()
    got = out.cpu()
    for i in range(n):
        m, nn, k = int(M[i]), int(N[i]), int(K[i])
        for h in range(H):
            a = A[h, a1[i]:a1[i] + m * k].float().reshape(m, k); b = B[h, a2[i]:a2[i] + nn * k].float().reshape(nn, k)
            ref = torch.softmax(a @ b.t() * scale, -1)
            seg = got[h, ao[i]:ao[i] + m * nn].float().reshape(m, nn)
            assert (seg - ref).abs().max().item() <= 1e-3, f"segment {i}, head {h}"
            hole = got[h, ao[i] + m * nn:ao[i + 1]]
            assert torch.isnan(hole).all(), f"the gap behind segment {i} was written"


def small_case(dev, rng, nseg=48):
    n = rng.integers(8, 200, nseg).astype(np.int64)
    n[:3] = [300, 5, 260]
    K = np.full(nseg, 64, np.int64)
    H, dtype = 2, torch.float16
    d1, do = int((n * K).sum()), int((n * n).sum())
    Md, Nd, Kd = dev_i64(n, dev), dev_i64(n, dev), dev_i64(K, dev)
    acc = [torch.empty(nseg + 1, dtype=torch.int64, device=dev) for _ in range(3)]
    A = torch.empty((H, d1), dtype=dtype, device=dev); B = torch.empty_like(A)
    out = torch.empty((H, do), dtype=dtype, device=dev)
    return n, K, H, dtype, d1, do, Md, Nd, Kd, acc, A, B, out


def test_the_call_is_one_kernel_node_in_a_captured_graph(dev):
    """Stream capture through the HIP runtime itself: the graph of one call has exactly one node, a kernel."""
    n, K, H, dtype, d1, do, Md, Nd, Kd, acc, A, B, out = small_case(dev, np.random.default_rng(30))
    capi.gemm_softmax_static(Md, Nd, Kd, A, B, out, H, d1, d1, do, 0.125, *acc)      # eager once, outside capture
    torch.cuda.synchronize()
    hip = ctypes.CDLL("libamdhip64.so.7")                      # the runtime this process already runs on
    for f in (hip.hipStreamBeginCapture, hip.hipStreamEndCapture, hip.hipGraphGetNodes, hip.hipGraphNodeGetType,
              hip.hipGraphDestroy):
        f.restype = ctypes.c_int
    stream = torch.cuda.Stream()
    handle = ctypes.c_void_p(stream.cuda_stream)
    graph = ctypes.c_void_p()
    with torch.cuda.stream(stream):
        assert hip.hipStreamBeginCapture(handle, 1) == 0        # thread-local capture mode
        capi.gemm_softmax_static(Md, Nd, Kd, A, B, out, H, d1, d1, do, 0.125, *acc)
        assert hip.hipStreamEndCapture(handle, ctypes.byref(graph)) == 0
    count = ctypes.c_size_t(0)
    assert hip.hipGraphGetNodes(graph, None, ctypes.byref(count)) == 0
    nodes = (ctypes.c_void_p * max(1, count.value))()
    assert hip.hipGraphGetNodes(graph, nodes, ctypes.byref(count)) == 0
    kinds = []
    for i in range(count.value):
        kind = ctypes.c_int(-1)
        assert hip.hipGraphNodeGetType(ctypes.c_void_p(nodes[i]), ctypes.byref(kind)) == 0
        kinds.append(kind.value)
    hip.hipGraphDestroy(graph)
    assert kinds == [0], f"expected one kernel node (type 0), got node types {kinds}"


def test_graph_replays_follow_the_lists(dev):
    rng = np.random.default_rng(31)
    nseg = 48
    n, K, H, dtype, d1, do, Md, Nd, Kd, acc, A, B, out = small_case(dev, rng, nseg)
    scale = 0.125

    def record():
        capi.gemm_softmax_static(Md, Nd, Kd, A, B, out, H, d1, d1, do, scale, *acc)

    record()                                                   # eager once, outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        record()
    for replay in range(3):
        order = rng.permutation(nseg)
        m = n[order]
        Ah, Bh = random_operands(m, m, K, H, dtype, seed=40 + replay)
        Md.copy_(dev_i64(m, dev)); Nd.copy_(Md)
        A.copy_(Ah); B.copy_(Bh)
        out.fill_(float("nan"))
        junk = torch.randn(1 << 20, device=dev).sum()          # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert_probs_close(out, oracle.per_segment_torch(Ah, Bh, m, m, K, scale), f"replay {replay}")
        assert torch.equal(acc[2].cpu(), torch.as_tensor(oracle.lists_to_accum(m, m, K)[2]))
        assert float(junk) == float(junk)


def test_unaligned_base_pointer_takes_the_element_wise_rows(dev):
    # A two bytes off a 16-byte boundary: no segment may use 16-byte operand loads, every workgroup walks its rows
    rng = np.random.default_rng(41)
    n = 30
    M = rng.integers(1, 60, n).astype(np.int64); N = rng.integers(1, 300, n).astype(np.int64)
    K = rng.choice(np.arange(8, 72, 8), n).astype(np.int64)
    H = 2
    A, B = random_operands(M, N, K, H, torch.float16, 8)
    d1, d2, do = int((M * K).sum()), int((N * K).sum()), int((M * N).sum())
    big = torch.zeros(H * d1 + 1, dtype=torch.float16, device=dev)
    big[1:] = A.reshape(-1).to(dev)
    out = torch.full((H, do), float("nan"), dtype=torch.float16, device=dev)
    capi.gemm_softmax_static(dev_i64(M, dev), dev_i64(N, dev), dev_i64(K, dev), big[1:], B.to(dev), out, H, d1, d2, do, 0.3)
    torch.cuda.synchronize()
    assert_probs_close(out, oracle.per_segment_torch(A, B, M, N, K, 0.3), "unaligned A")


def test_given_prefix_sums_that_overlap_are_rejected(dev):
    M = np.array([20, 30], np.int64); N = np.array([24, 36], np.int64); K = np.array([32, 32], np.int64)
    a1 = np.array([0, 640, 1600], np.int64); a2 = np.array([0, 768, 1920], np.int64)
    ao = np.array([0, 400, 1560], np.int64)                # segment 0 needs 480 results, its slot holds 400
    A = torch.randn((1, 1600)).half(); B = torch.randn((1, 1920)).half()
    out = torch.full((1, 1560), float("nan"), dtype=torch.float16, device=dev)
    capi.gemm_softmax_static(dev_i64(M, dev), dev_i64(N, dev), dev_i64(K, dev), A.to(dev), B.to(dev), out, 1, 1600, 1920, 1560,
                             1.0, dev_i64(a1, dev), dev_i64(a2, dev), dev_i64(ao, dev), mode=capi.META_GIVEN)
    torch.cuda.synchronize()
    assert torch.isnan(out).all()
    info, st = capi.static_read(raise_on_bad=False)
    assert st == 5 and info.bad_segments >= 1


def test_many_heads_up_to_the_pair_limit_and_beyond(dev):
    # 200 segments x 5 heads = 1000 pairs: the single launch; x 6 heads: scheduler + plan-driven kernels; same results
    rng = np.random.default_rng(43)
    n = 200
    M = rng.integers(1, 70, n).astype(np.int64); N = rng.integers(1, 130, n).astype(np.int64)
    K = rng.choice(np.arange(8, 72, 8), n).astype(np.int64)
    for H in (5, 6):
        run_static(dev, M, N, K, H, torch.bfloat16, 0.21, seed=H)
