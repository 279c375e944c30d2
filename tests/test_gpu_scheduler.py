"""Device-side scheduler against the oracle: offsets and lists bit-exact, work
items an exact cover, bad metadata rejected (all through the C ABI)."""
import numpy as np
import pytest
import torch

import oracle
from blockedattention_amd import capi, workloads
from _util import dev_i64, make_plan

pytestmark = pytest.mark.gpu


def expected_items(M, N, K):
    """Host restatement of the plan's classification for lists-only metadata."""
    M = np.asarray(M); N = np.asarray(N); K = np.asarray(K)
    a1, a2, _ = oracle.lists_to_accum(M, N, K)
    aligned = ((K | a1[:-1] | a2[:-1]) & 7) == 0
    strips = np.where(N >= 1, -(-M // 16), 0)
    pack = np.zeros(len(M), np.int64)
    for w0 in range(0, len(M), 16):
        i = w0
        end = min(w0 + 16, len(M))
        while i < end:
            ln = sm = sn = 0
            while i + ln < end:
                g = i + ln
                if M[g] < 1 or N[g] < 1 or not aligned[g] or K[g] != K[i] or K[i] < 1 or not aligned[i]:
                    break
                if sm + M[g] > 16 or sn + N[g] > 16:
                    break
                sm += M[g]; sn += N[g]; ln += 1
            if ln >= 2:
                pack[i] = ln; pack[i + 1:i + ln] = -1; i += ln
            else:
                i += 1
    ok = aligned & (pack == 0)
    return {
        "gemm_items": int((strips * -(-N // 256))[ok & (N > 256)].sum()),
        "strip_items": int(strips[ok & (N <= 256)].sum()),
        "split_items": int(strips[ok & (N > 256) & (N <= 4096)].sum()),
        "wide_items": int(strips[ok & (N > 4096)].sum()),
        "pack_items": int((pack > 0).sum()),
        "slow_items": int(strips[~aligned].sum()),
        "total_rows": int(M[N >= 1].sum()),
    }


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5])
def test_offsets_bit_exact_and_items_cover(dev, cfg):
    w = workloads.make(cfg)
    plan = make_plan(dev, w.M, w.N, w.K)
    a1, a2, ao = oracle.lists_to_accum(w.M, w.N, w.K)
    for got, ref in zip(plan.keep[3:], (a1, a2, ao)):
        assert got.dtype == torch.int64 and np.array_equal(got.cpu().numpy(), ref)
    info = plan.info.as_dict()
    assert (info["Dm1"], info["Dm2"], info["Dout"]) == (w.Dm1, w.Dm2, w.Dout)
    assert (info["max_M"], info["max_N"], info["max_K"]) == (w.M.max(), w.N.max(), w.K.max())
    for k, v in expected_items(w.M, w.N, w.K).items():
        assert info[k] == v, (k, info[k], v)
    assert info["bad_segments"] == 0


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5])
def test_lists_from_prefix_sums_are_exact(dev, cfg):
    w = workloads.make(cfg)
    a1, a2, ao = [dev_i64(a, dev) for a in oracle.lists_to_accum(w.M, w.N, w.K)]
    M = torch.full((w.nseg,), -7, dtype=torch.int64, device=dev); N = M.clone(); K = M.clone()
    plan = capi.plan_gemm(w.nseg, dev, M, N, K, a1, a2, ao, mode=capi.META_FROM_ACCUM)
    info = plan.read()
    assert np.array_equal(M.cpu().numpy(), w.M) and np.array_equal(N.cpu().numpy(), w.N)
    assert np.array_equal(K.cpu().numpy(), w.K)
    assert (info.Dm1, info.Dm2, info.Dout, info.bad_segments) == (w.Dm1, w.Dm2, w.Dout, 0)


def test_lists_from_prefix_sums_large_and_degenerate(dev):
    M = np.array([4097, 99991, 16777217, 3, 0, 1 << 15]); N = np.array([4095, 7, 3, 16777219, 0, 1 << 14])
    K = np.array([127, 9989, 5, 2, 0, 1 << 14])
    a = [dev_i64(x, dev) for x in oracle.lists_to_accum(M, N, K)]
    m = torch.empty(6, dtype=torch.int64, device=dev); n = m.clone(); k = m.clone()
    info = capi.plan_gemm(6, dev, m, n, k, *a, mode=capi.META_FROM_ACCUM).read()
    assert info.bad_segments == 0
    assert np.array_equal(m.cpu().numpy(), M) and np.array_equal(n.cpu().numpy(), N) and np.array_equal(k.cpu().numpy(), K)
    # inconsistent areas are rejected, and reported as -1 like the oracle does
    a1, a2, ao = dev_i64([0, 6, 12], dev), dev_i64([0, 10, 20], dev), dev_i64([0, 14, 29], dev)
    m = torch.empty(2, dtype=torch.int64, device=dev); n = m.clone(); k = m.clone()
    plan = capi.plan_gemm(2, dev, m, n, k, a1, a2, ao, mode=capi.META_FROM_ACCUM)
    info = plan.read(raise_on_bad=False)
    om, on, ok, obad = oracle.accum_to_lists([0, 6, 12], [0, 10, 20], [0, 14, 29])
    assert info.bad_segments == obad == 1
    assert np.array_equal(m.cpu().numpy(), om) and np.array_equal(k.cpu().numpy(), ok)


def test_segment_areas_of_2_to_the_30_elements_are_rejected(dev):
    # every dimension is admissible, one area is not: the kernels address a segment with 32-bit byte offsets, so
    # M K, N K and M N of a segment stay below 2^30 elements -- from lists and from prefix sums alike
    for M, N, K in (([40000, 8], [40000, 8], [8, 8]), ([1 << 20, 8], [16, 8], [1 << 10, 8]), ([16, 8], [1 << 20, 8], [1 << 10, 8])):
        plan = make_plan(dev, np.array(M), np.array(N), np.array(K), read=False)
        assert plan.read(raise_on_bad=False).bad_segments == 1
        a = [dev_i64(x, dev) for x in oracle.lists_to_accum(np.array(M), np.array(N), np.array(K))]
        m = torch.empty(2, dtype=torch.int64, device=dev); n = m.clone(); k = m.clone()
        plan = capi.plan_gemm(2, dev, m, n, k, *a, mode=capi.META_FROM_ACCUM)
        assert plan.read(raise_on_bad=False).bad_segments == 1
    # just below the limit is fine
    plan = make_plan(dev, np.array([32767]), np.array([32768]), np.array([8]), read=False)
    assert plan.read(raise_on_bad=False).bad_segments == 0


def test_more_segments_than_one_scheduler_pass(dev):
    rng = np.random.default_rng(7)
    B = 5000
    M = rng.integers(0, 40, B); N = rng.integers(0, 40, B); K = rng.choice([0, 8, 16, 24, 61], B)
    plan = make_plan(dev, M, N, K)
    a1, a2, ao = oracle.lists_to_accum(M, N, K)
    for got, ref in zip(plan.keep[3:], (a1, a2, ao)):
        assert np.array_equal(got.cpu().numpy(), ref)
    info = plan.info.as_dict()
    for k, v in expected_items(M, N, K).items():
        assert info[k] == v, (k, info[k], v)


def test_bad_metadata_is_rejected_and_kernels_refuse_to_run(dev):
    M = dev_i64([4, -1, 3], dev); N = dev_i64([4, 2, 3], dev); K = dev_i64([8, 8, 8], dev)
    plan = capi.plan_gemm(3, dev, M, N, K, mode=capi.META_FROM_LISTS)
    with pytest.raises(capi.BlockedAttentionError, match="metadata"):
        plan.read()
    info = plan.read(raise_on_bad=False)
    assert info.bad_segments == 1
    # given both halves, a prefix sum too small for its segment is rejected
    a1 = dev_i64([0, 32, 40], dev); a2 = dev_i64([0, 32, 64], dev); ao = dev_i64([0, 16, 32], dev)
    plan = capi.plan_gemm(2, dev, dev_i64([4, 4], dev), dev_i64([4, 4], dev), dev_i64([8, 8], dev), a1, a2, ao,
                          mode=capi.META_GIVEN)
    assert plan.read(raise_on_bad=False).bad_segments == 1
    out = torch.full((1, 32), 7.0, dtype=torch.float16, device=dev)
    A = torch.zeros((1, 40), dtype=torch.float16, device=dev); B = torch.zeros((1, 64), dtype=torch.float16, device=dev)
    capi.varlen_gemm(plan, A, B, out, 1, 40, 64, 32)
    torch.cuda.synchronize()
    assert (out == 7.0).all() and plan.read(raise_on_bad=False).run_errors == 1


def test_size_mismatch_makes_kernels_refuse(dev):
    plan = make_plan(dev, [4], [4], [8])
    out = torch.full((1, 16), 7.0, dtype=torch.float16, device=dev)
    A = torch.zeros((1, 64), dtype=torch.float16, device=dev)
    capi.varlen_gemm(plan, A, A, out, 1, 64, 64, 16)       # Dm1 should be 32
    torch.cuda.synchronize()
    assert (out == 7.0).all() and plan.read(raise_on_bad=False).run_errors == 1


def test_softmax_plan_offsets(dev):
    rows = [33, 99, 64, 0, 5]; cols = [64, 64, 64, 7, 0]
    acc = torch.empty(6, dtype=torch.int64, device=dev)
    plan = capi.plan_softmax(5, dev, dev_i64(rows, dev), dev_i64(cols, dev), acc)
    info = plan.read()
    assert np.array_equal(acc.cpu().numpy(), oracle.softmax_accum(rows, cols))
    assert info.Dout == 12544 and info.total_rows == 196


def test_empty_batch(dev):
    e = torch.empty(0, dtype=torch.int64, device=dev)
    a = [torch.full((1,), -1, dtype=torch.int64, device=dev) for _ in range(3)]
    info = capi.plan_gemm(0, dev, e, e, e, *a, mode=capi.META_FROM_LISTS).read()
    assert (info.nseg, info.Dm1, info.Dm2, info.Dout, info.gemm_items) == (0, 0, 0, 0, 0)
    assert all(int(t[0]) == 0 for t in a)


def test_row_block_prefixes_of_the_attention_work_list(dev):
    # Behind the work lists the plan keeps, for blocks of 64 and of 128 rows, how many row blocks the segments
    # before each segment have (every segment with rows counts, whatever its N and K); entry nseg = total.
    rng = np.random.default_rng(11)
    for nseg in (1, 63, 300, 2500):
        M = rng.integers(0, 700, nseg); N = rng.integers(0, 40, nseg); K = rng.choice([0, 8, 64], nseg)
        plan = make_plan(dev, M, N, K, read=False)
        cap = (nseg + 4) & ~3
        words = plan.buf.cpu().numpy()[256 + 6 * 48 * cap:].view(np.int32)
        for which, rows in ((0, 64), (1, 128)):
            blocks = np.where(M >= 1, (M + rows - 1) // rows, 0)
            want = np.concatenate([[0], np.cumsum(blocks)]).astype(np.int32)
            got = words[which * (cap + 4): which * (cap + 4) + nseg + 1]
            assert np.array_equal(got, want), (nseg, rows)


def _mini(M, N, K):
    tiles = 2 * ((N + 31) // 32); blocks = tiles * ((K + 31) // 32)
    return (M >= 1) & (M <= 64) & (N >= 2) & (blocks >= 1) & (blocks <= 16) & (tiles <= 8)


def test_main_strip_list_is_a_permutation_in_work_buckets(dev):
    # Batches of 65 to 256 segments keep the main strip launch's list in eight buckets of decreasing work
    # (16-row strips x column tiles / 8, clipped at 7), in segment order inside a bucket; every other batch
    # keeps segment order.  The mini segments of the list (at most 64 rows, B_g of at most 16 KiB, at most eight
    # column tiles) are kept apart, from the end of the list's array backwards, in segment order.  Together the
    # two parts hold each segment of the list exactly once.
    rec = np.dtype([("o1", "<i8"), ("o2", "<i8"), ("oo", "<i8"), ("M", "<i4"), ("N", "<i4"), ("K", "<i4"),
                    ("pack", "<i4"), ("kind", "<i4"), ("index", "<i4")])
    rng = np.random.default_rng(5)
    for nseg in (40, 200, 256, 300):
        M = rng.integers(17, 130, nseg); N = rng.integers(17, 130, nseg); K = np.full(nseg, 64)
        plan = make_plan(dev, M, N, K)
        mini = _mini(M, N, K)
        assert 0 < mini.sum() < nseg
        assert plan.info.list_small == nseg - mini.sum() and plan.info.list_mini == mini.sum()
        cap = (nseg + 4) & ~3
        raw = plan.buf.cpu().numpy()
        arr = raw[256 + cap * 48: 256 + 2 * cap * 48].view(rec)
        lst = arr[:plan.info.list_small]
        tail = arr[::-1][:plan.info.list_mini]
        assert sorted(lst["index"].tolist() + tail["index"].tolist()) == list(range(nseg))
        assert np.array_equal(tail["index"], np.nonzero(mini)[0])
        for part in (lst, tail):
            assert np.array_equal(part["M"], M[part["index"]]) and np.array_equal(part["N"], N[part["index"]])
        others = np.nonzero(~mini)[0]
        bucket = np.minimum(7, ((M + 15) // 16) * (2 * ((N + 31) // 32)) // 8)[others]
        if 64 < nseg <= 256:
            want = others[np.argsort(-bucket, kind="stable")]
        else:
            want = others
        assert np.array_equal(lst["index"], want), nseg


def test_summary_through_a_mailbox_and_through_caller_memory(dev):
    # the scheduler hands the summary to the host in pinned memory (ticket behind it); the host spins, no copy and
    # no stream synchronisation.  And ba_plan_read through a pinned buffer of the caller.  Both equal ba_plan_read.
    rng = np.random.default_rng(12)
    mailbox = torch.zeros(capi.MAILBOX_BYTES, dtype=torch.uint8).pin_memory()
    staging = torch.zeros(256, dtype=torch.uint8).pin_memory()
    for ticket, nseg in enumerate((5, 300, 2000), start=1):
        M = rng.integers(0, 300, nseg); N = rng.integers(0, 300, nseg); K = 8 * rng.integers(0, 17, nseg)
        Md, Nd, Kd = dev_i64(M, dev), dev_i64(N, dev), dev_i64(K, dev)
        acc = [torch.empty(nseg + 1, dtype=torch.int64, device=dev) for _ in range(3)]
        plan = capi.plan_gemm(nseg, dev, Md, Nd, Kd, *acc, mode=capi.META_FROM_LISTS, mailbox=mailbox, ticket=ticket)
        got = plan.wait(mailbox, ticket).as_dict()
        want = plan.read().as_dict()
        assert got == want and got["nseg"] == nseg
        assert plan.read_into(staging).as_dict() == want
    # a ticket nobody writes: the wait gives up
    with pytest.raises(capi.BlockedAttentionError, match="launch"):
        plan.wait(mailbox, 999, timeout_us=20_000)


def test_prefix_sums_with_one_empty_dimension(dev):
    # M = 0 (or N = 0, or K = 0) leaves a single non-zero area: the product of the other two dimensions, whose
    # split changes no result.  The scheduler and the oracle take the same convention and accept the batch.
    M = np.array([0, 5, 7, 0, 3]); N = np.array([4, 0, 6, 0, 2]); K = np.array([8, 8, 0, 0, 16])
    a1, a2, ao = oracle.lists_to_accum(M, N, K)
    Mo, No, Ko, bad = oracle.accum_to_lists(a1, a2, ao)
    assert bad == 0
    assert np.array_equal(Mo * Ko, M * K) and np.array_equal(No * Ko, N * K) and np.array_equal(Mo * No, M * N)
    lists = [torch.empty(5, dtype=torch.int64, device=dev) for _ in range(3)]
    plan = capi.plan_gemm(5, dev, *lists, dev_i64(a1, dev), dev_i64(a2, dev), dev_i64(ao, dev), mode=capi.META_FROM_ACCUM)
    info = plan.read()
    assert info.bad_segments == 0
    got = [t.cpu().numpy() for t in lists]
    assert np.array_equal(got[0], Mo) and np.array_equal(got[1], No) and np.array_equal(got[2], Ko)


def test_batches_beyond_the_32_bit_work_counts_are_rejected(dev):
    # three segments of 2^30 - 1 rows each: every one is admissible, their row count together is not
    big = (1 << 30) - 1
    M = np.array([big, big, big]); N = np.array([1, 1, 1]); K = np.array([0, 0, 0])
    plan = make_plan(dev, M, N, K, read=False)
    assert plan.read(raise_on_bad=False).bad_segments >= 1
    plan = make_plan(dev, M[:1], N[:1], K[:1], read=False)
    assert plan.read(raise_on_bad=False).bad_segments == 0
