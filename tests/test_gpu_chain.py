"""GPU parity of chained matmuls (consecutive one- or two-row Q4_K / Q5_K entries of
gllmq_quantized_matmul_batch run as one launch whose loader waves go straight on from one matrix's
weights to the next one's; entries flagged GLLMQ_DESC_AFTER_PREVIOUS wait inside the launch for the
entry before them) against the oracle, through the C ABI.  The reference launches a decode step
once (src/compat/hip_backend.rs:224-236) and its ops read each other's outputs
(build_graph.inc.rs:1960-1999): the dependent case here feeds every matmul the output of the one
before.  Same bar as the other matmul tests; against the one-launch-per-entry form (option
"chain" = 0) the results are equal bit for bit."""
import numpy as np
import pytest

from gllm_amd.synth import random_activations, random_weight
from tests.test_gpu_parity import check_close

pytestmark = pytest.mark.gpu

Q4_K, Q5_K, Q8_0 = 12, 13, 8


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def cus(torch):
    return torch.cuda.get_device_properties(0).multi_processor_count


def dev_weight(torch, w):
    return torch.from_numpy(np.asarray(w).view(np.uint8).reshape(-1)).cuda()


def run_batch(hip, torch, entries, after_previous):
    """entries: [(w_dev, x_dev, y_dev, dtype, m, n, k)]"""
    batch = hip.make_batch(entries, after_previous=after_previous)
    hip.run_batch(batch, 0, len(entries))
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype,m", [(Q4_K, 1), (Q5_K, 1), (Q4_K, 2), (Q5_K, 2), (Q8_0, 1), (Q8_0, 2)])
def test_independent_entries_of_different_heights(torch, oracle, dtype, m):
    """The matmuls of a decoder layer that share K: different numbers of weight rows, so different
    tile heights and numbers of workgroups per entry, one launch."""
    from gllm_amd.backend import HipBackend
    # (single launches in the streamed form throughout: by default a short Q5_K entry would take the GEMV)
    hip, plain = HipBackend(0), HipBackend(0, options={"chain": 0, "mm8s_all": 1})
    c, k = cus(torch), 4096
    ns = [24 * c, 16 * c, 112 * c + 5, 8 * c, 56 * c + 31]
    host = [(random_weight(dtype, n, k, seed=i), random_activations(m, k, seed=10 + i)) for i, n in enumerate(ns)]
    outs = []
    for backend in (hip, plain):
        entries = [(dev_weight(torch, w), torch.from_numpy(x).cuda(), torch.full((m, n), float("nan"), device="cuda"), dtype, m, n, k)
                   for (w, x), n in zip(host, ns)]
        print(f"chain: independent dtype={dtype} m={m} chain={backend is hip}", flush=True)
        run_batch(backend, torch, entries, after_previous=None)
        assert backend.last_kernel_name().startswith("gq_mm8c_") == (backend is hip), backend.last_kernel_name()
        outs.append([e[2].cpu().numpy() for e in entries])
    for i, ((w, x), n) in enumerate(zip(host, ns)):
        want = oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=16)
        check_close(outs[0][i], want, f"entry {i}")
        assert np.array_equal(outs[0][i].view(np.uint32), outs[1][i].view(np.uint32)), f"entry {i}: chained and single launches differ"


@pytest.mark.parametrize("dtype,m", [(Q4_K, 1), (Q5_K, 2), (Q8_0, 1)])
def test_entries_with_few_weight_rows_join_the_chain(torch, oracle, dtype, m):
    """Separate Q, K and V projections of a grouped-query layer (K and V have a quarter of the rows)
    and smaller ones still, down to fewer rows than CUs: tiles of a few rows, workgroups without a
    share of an entry.  One launch; against the oracle (a launch of its own would split K across
    workgroups for such entries and add up in another order)."""
    from gllm_amd.backend import HipBackend
    hip = HipBackend(0)
    c, k = cus(torch), 2048
    ns = [16 * c, 4 * c, 4 * c, c + 44, 100, 33, 1, 9 * c]
    host = [(random_weight(dtype, n, k, seed=40 + i), random_activations(m, k, seed=50 + i)) for i, n in enumerate(ns)]
    entries = [(dev_weight(torch, w), torch.from_numpy(x).cuda(), torch.full((m * n + 64,), float("nan"), device="cuda"), dtype, m, n, k)
               for (w, x), n in zip(host, ns)]
    for e, n in zip(entries, ns):
        e[2][m * n:] = 7.0
    print(f"chain: small entries dtype={dtype} m={m}", flush=True)
    run_batch(hip, torch, [(w, x, y[:m * n], dt, mm, n, kk) for (w, x, y, dt, mm, n, kk) in entries], after_previous=None)
    assert hip.last_kernel_name().startswith("gq_mm8c_"), hip.last_kernel_name()
    for i, ((w, x), n) in enumerate(zip(host, ns)):
        got = entries[i][2].cpu().numpy()
        assert np.all(got[m * n:] == 7.0), f"entry {i}: write past the output"
        check_close(got[:m * n].reshape(m, n), oracle.quantized_matmul(w, x, dtype, m, n, k, acc=oracle.ACC_F64, threads=8), f"entry {i}")


@pytest.mark.parametrize("dtype,m", [(Q4_K, 1), (Q5_K, 1), (Q4_K, 2), (Q8_0, 1)])
def test_entries_that_share_their_activations(torch, oracle, dtype, m):
    """Q, K and V read the same x, gate and up another, a last entry the first again: a workgroup
    prepares an x once for the entries in a row that share it (also one that skipped an entry it
    has no rows of).  Equal to single launches bit for bit, and against the oracle."""
    from gllm_amd.backend import HipBackend
    hip, plain = HipBackend(0), HipBackend(0, options={"chain": 0, "mm8s_all": 1})
    c, k = cus(torch), 4096
    ns = [16 * c, 4 * c, c // 2, 4 * c + 3, 56 * c, 56 * c, 16 * c]
    which_x = [0, 0, 0, 0, 1, 1, 0]
    xs_host = [random_activations(m, k, seed=40 + i) for i in range(2)]
    ws_host = [random_weight(dtype, n, k, seed=50 + i) for i, n in enumerate(ns)]
    outs = []
    for backend in (hip, plain):
        xs = [torch.from_numpy(x).cuda() for x in xs_host]
        entries = [(dev_weight(torch, w), xs[xi], torch.full((m, n), float("nan"), device="cuda"), dtype, m, n, k)
                   for w, n, xi in zip(ws_host, ns, which_x)]
        print(f"chain: shared x dtype={dtype} m={m} chain={backend is hip}", flush=True)
        run_batch(backend, torch, entries, after_previous=None)
        if backend is hip:
            assert backend.last_kernel_name().startswith("gq_mm8c_"), backend.last_kernel_name()
        outs.append([e[2].cpu().numpy() for e in entries])
    for i, (w, n, xi) in enumerate(zip(ws_host, ns, which_x)):
        want = oracle.quantized_matmul(w, xs_host[xi], dtype, m, n, k, acc=oracle.ACC_F64, threads=16)
        check_close(outs[0][i], want, f"entry {i}")
        if n >= 4 * c:  # (fewer rows: a launch of its own splits K across workgroups, another order of sums)
            assert np.array_equal(outs[0][i].view(np.uint32), outs[1][i].view(np.uint32)), f"entry {i}: chained and single launches differ"


def test_every_entry_reads_the_output_of_the_one_before(torch, oracle):
    """y0 = W0 x, y1 = W1 y0, ...: every entry waits inside the launch for the workgroups of the one
    before it and reads what they stored.  Each step is checked against the oracle on the input
    the GPU actually had; twice, so the counters are seen to be back at zero."""
    from gllm_amd.backend import HipBackend
    hip = HipBackend(0, options={"chain_dependent": 1})  # by default such an entry starts a launch of its own
    k = 4096
    steps = 7
    ws = [random_weight(Q4_K, k, k, seed=20 + i) for i in range(steps)]
    wd = [dev_weight(torch, w) for w in ws]
    for attempt in range(2):
        x0 = (random_activations(1, k, seed=attempt) * 0.5).astype(np.float32)
        bufs = [torch.from_numpy(x0).cuda()] + [torch.full((1, k), float("nan"), device="cuda") for _ in range(steps)]
        entries = [(wd[i], bufs[i], bufs[i + 1], Q4_K, 1, k, k) for i in range(steps)]
        print(f"chain: dependent entries, attempt {attempt}", flush=True)
        run_batch(hip, torch, entries, after_previous=lambda i: i > 0)
        assert hip.last_kernel_name().startswith("gq_mm8c_q4k")
        got = [b.cpu().numpy() for b in bufs]
        for i in range(steps):
            assert np.isfinite(got[i + 1]).all(), f"step {i}: an entry started before its input was complete"
            # the outputs grow by about sqrt(k) * |w| per step: scale the next input down on the host side of the check only
            want = oracle.quantized_matmul(ws[i], got[i], Q4_K, 1, k, k, acc=oracle.ACC_F64, threads=16)
            check_close(got[i + 1], want, f"attempt {attempt} step {i}")


def test_long_batch_splits_into_chains_and_mixes_with_other_kernels(torch, oracle):
    """Seventy entries (more than one launch holds), every third one dependent, with a Q6_K matmul
    and a 16-row GEMM in between that are not for the chain kernel; with dependent entries kept in
    the chains and (the default) starting launches of their own."""
    from gllm_amd.backend import HipBackend
    for options in ({"chain_dependent": 1}, {}):
        many_entries(HipBackend(0, options=options), torch, oracle)


def many_entries(hip, torch, oracle):
    c, k = cus(torch), 2048
    n = 9 * c + 3
    w = random_weight(Q4_K, n, k, seed=1)
    w6 = random_weight(14, 300, k, seed=2)
    wd, w6d = dev_weight(torch, w), dev_weight(torch, w6)
    xs = [random_activations(1, k, seed=100 + i) for i in range(70)]
    x16 = random_activations(16, k, seed=3)
    entries, kinds = [], []
    for i, x in enumerate(xs):
        entries.append((wd, torch.from_numpy(x).cuda(), torch.full((1, n), float("nan"), device="cuda"), Q4_K, 1, n, k))
        kinds.append(("q4", i))
        if i == 40:
            entries.append((w6d, torch.from_numpy(xs[0]).cuda(), torch.full((1, 300), float("nan"), device="cuda"), 14, 1, 300, k))
            kinds.append(("q6", 0))
            entries.append((wd, torch.from_numpy(x16).cuda(), torch.full((16, n), float("nan"), device="cuda"), Q4_K, 16, n, k))
            kinds.append(("gemm", 0))
    print("chain: seventy entries", flush=True)
    run_batch(hip, torch, entries, after_previous=lambda i: i % 3 == 1)
    want1 = {i: oracle.quantized_matmul(w, xs[i], Q4_K, 1, n, k, acc=oracle.ACC_F64, threads=16) for i in (0, 31, 32, 40, 41, 69)}
    for e, (kind, i) in zip(entries, kinds):
        got = e[2].cpu().numpy()
        assert np.isfinite(got).all()
        if kind == "q4" and i in want1:
            check_close(got, want1[i], f"entry {i}")
        elif kind == "q6":
            check_close(got, oracle.quantized_matmul(w6, xs[0], 14, 1, 300, k, acc=oracle.ACC_F64, threads=4), "the Q6_K entry")
        elif kind == "gemm":
            check_close(got, oracle.quantized_matmul(w, x16, Q4_K, 16, n, k, acc=oracle.ACC_F64, threads=16), "the 16-row entry")


def test_a_wait_that_runs_out_is_reported_and_the_launch_still_ends(torch):
    """With no repeats allowed a wave that finds its activations not yet posted gives up at once:
    the launch ends (nothing hangs), the next batch call reports the failure once, and the call
    after that works again."""
    from gllm_amd.backend import BackendError, HipBackend
    hip = HipBackend(0, options={"chain_spin_limit": 0, "chain_dependent": 1})
    c, k = cus(torch), 4096
    n = 56 * c
    wd = dev_weight(torch, random_weight(Q4_K, n, k, seed=1))
    x = torch.from_numpy(random_activations(1, k, seed=2)).cuda()
    ys = [torch.empty(1, n, device="cuda") for _ in range(6)]
    entries = [(wd, x if i == 0 else ys[i - 1], ys[i], Q4_K, 1, n, k) for i in range(6)]  # each reads the first k outputs of the one before
    print("chain: waits that run out", flush=True)
    run_batch(hip, torch, entries, after_previous=lambda i: i > 0)
    assert hip.last_kernel_name().startswith("gq_mm8c_q4k")
    with pytest.raises(BackendError, match="timed out"):
        run_batch(hip, torch, entries, after_previous=lambda i: i > 0)
    hip.set_option("chain_spin_limit", 1 << 20)
    run_batch(hip, torch, entries, after_previous=lambda i: i > 0)  # the error was reported once; this one runs
    run_batch(hip, torch, entries, after_previous=lambda i: i > 0)


def test_a_wait_that_runs_out_can_be_asked_for(torch):
    """gllmq_chain_status after a synchronisation: set once by the launch whose wait ran out, set back
    by the look, so that the next batch call has nothing to report."""
    from gllm_amd.backend import HipBackend
    hip = HipBackend(0, options={"chain_spin_limit": 0, "chain_dependent": 1})
    c, k = cus(torch), 4096
    n = 56 * c
    wd = dev_weight(torch, random_weight(Q4_K, n, k, seed=1))
    x = torch.from_numpy(random_activations(1, k, seed=2)).cuda()
    ys = [torch.empty(1, n, device="cuda") for _ in range(6)]
    entries = [(wd, x if i == 0 else ys[i - 1], ys[i], Q4_K, 1, n, k) for i in range(6)]
    assert not hip.chain_status()
    print("chain: status after a wait that ran out", flush=True)
    run_batch(hip, torch, entries, after_previous=lambda i: i > 0)
    assert hip.chain_status() and not hip.chain_status()
    hip.set_option("chain_spin_limit", 1 << 20)
    run_batch(hip, torch, entries, after_previous=lambda i: i > 0)  # nothing left to report
    assert not hip.chain_status()


def test_a_captured_batch_replays_like_the_eager_one(torch, oracle):
    """A batch with a chained launch (Q, K, V on one x), an entry that waits for it, independent entries
    of other kinds and an entry of sixteen rows, captured into a graph: every replay gives the bits
    of the eager call on the same inputs (a captured batch runs its kernels as ordinary launches)."""
    from gllm_amd.backend import HipBackend
    hip = HipBackend(0)
    c, k = cus(torch), 2048
    ns = [16 * c, 4 * c, 4 * c, 12 * c, 9 * c, 8 * c]
    dts = [Q4_K, Q4_K, Q4_K, Q4_K, 14, Q5_K]
    ms = [1, 1, 1, 1, 1, 16]
    ws = [dev_weight(torch, random_weight(dt, n, k, seed=70 + i)) for i, (dt, n) in enumerate(zip(dts, ns))]
    x1, x16 = torch.empty(1, k, device="cuda"), torch.empty(16, k, device="cuda")
    def outputs():
        return [torch.full((m, n), float("nan"), device="cuda") for m, n in zip(ms, ns)]
    got, want = outputs(), outputs()
    def entries(ys):
        return [(w, x16 if m == 16 else x1, y, dt, m, n, k) for w, y, dt, m, n in zip(ws, ys, dts, ms, ns)]
    flags = lambda i: i == 3  # the fourth entry starts after the chain of the first three
    eager = hip.make_batch(entries(want), after_previous=flags)
    captured = hip.make_batch(entries(got), after_previous=flags)
    x1.copy_(torch.from_numpy(random_activations(1, k, seed=1)).cuda())
    x16.copy_(torch.from_numpy(random_activations(16, k, seed=2)).cuda())
    hip.run_batch(captured, 0, len(ns))  # once eagerly: the stream's scratch exists before the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    print("chain: a batch inside a graph", flush=True)
    with torch.cuda.stream(side):
        hip.run_batch(captured, 0, len(ns))
        side.synchronize()
        graph.capture_begin()
        hip.run_batch(captured, 0, len(ns))
        graph.capture_end()
    torch.cuda.synchronize()
    for rep in range(3):
        x1.copy_(torch.from_numpy(random_activations(1, k, seed=10 + rep)).cuda())
        x16.copy_(torch.from_numpy(random_activations(16, k, seed=20 + rep)).cuda())
        for y in got:
            y.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        hip.run_batch(eager, 0, len(ns))
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert not bool(torch.isnan(b).any())
            assert torch.equal(a.view(torch.int32), b.view(torch.int32)), f"replay {rep}, entry {i}"
    x = x1.cpu().numpy()
    check_close(got[0].cpu().numpy(), oracle.quantized_matmul(random_weight(Q4_K, ns[0], k, seed=70), x, Q4_K, 1, ns[0], k,
                                                               acc=oracle.ACC_F64, threads=16), "entry 0 of the last replay")


def test_the_weight_prefetch_beside_dependent_launches_changes_no_bit(torch):
    """Option "prefetch": a launch on a stream of the context's own reads the weights of each
    dependent entry into the memory-side cache while the entry before it runs (it waits for that
    launch's announcement, bounded by a time-out, and writes nothing).  Same outputs bit for bit as
    without it, over a sequence in which every matmul reads the output of the one before; large and
    small matrices (entries under the size threshold are left out of the prefetch), twice, and
    ordinary calls on the stream afterwards."""
    from gllm_amd.backend import HipBackend
    with_it, without = HipBackend(0, options={"prefetch": 1}), HipBackend(0)
    k = 4096
    ns = [4096, 4096, 14336]
    ws = [random_weight(Q4_K, ns[0], k, seed=70), random_weight(Q4_K, ns[1], k, seed=71), random_weight(Q4_K, ns[2], k, seed=72)]
    wd = [dev_weight(torch, w) for w in ws]
    for attempt in range(2):
        x0 = (random_activations(1, k, seed=80 + attempt) * 0.5).astype(np.float32)
        outs = []
        for backend in (with_it, without):
            bufs = [torch.from_numpy(x0).cuda(), torch.full((1, ns[0]), float("nan"), device="cuda"),
                    torch.full((1, ns[1]), float("nan"), device="cuda"), torch.full((1, ns[2]), float("nan"), device="cuda")]
            entries = [(wd[i], bufs[i], bufs[i + 1], Q4_K, 1, ns[i], k) for i in range(3)]
            print(f"prefetch: attempt {attempt} prefetch={backend is with_it}", flush=True)
            run_batch(backend, torch, entries, after_previous=lambda i: i > 0)
            outs.append([b.cpu().numpy() for b in bufs[1:]])
        for a, b in zip(*outs):
            assert np.isfinite(a).all()
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # an ordinary call behind the batches on the same stream
    x = torch.from_numpy(random_activations(1, k, seed=90)).cuda()
    ya, yb = torch.empty(1, ns[2], device="cuda"), torch.empty(1, ns[2], device="cuda")
    with_it.quantized_matmul(wd[2], x, ya, Q4_K, 1, ns[2], k)
    without.quantized_matmul(wd[2], x, yb, Q4_K, 1, ns[2], k)
    torch.cuda.synchronize()
    assert torch.equal(ya.view(torch.int32), yb.view(torch.int32))


@pytest.mark.parametrize("dtype,m", [(Q4_K, 1), (Q5_K, 2), (Q8_0, 1)])
def test_open_requests_per_loader_change_no_bit(torch, dtype, m):
    """By default a loader of the chained launch keeps one item open on entries of full tiles and
    two on entries of low tiles or paired blocks; whatever number it is told to keep, and however
    often it stands before a taken slot and counts its open requests in there, the results are
    the same bits."""
    from gllm_amd.backend import HipBackend
    c, k = cus(torch), 4096
    ns = [24 * c, 16 * c, 112 * c + 5, 8 * c, 56 * c + 31, 16 * c, 24 * c + 3]
    host = [(random_weight(dtype, n, k, seed=40 + i), random_activations(m, k, seed=50 + i)) for i, n in enumerate(ns)]
    outs = []
    for depth in (0, 1, 2, 3, 4):
        backend = HipBackend(0, options={"mm8s_depth": depth})
        entries = [(dev_weight(torch, w), torch.from_numpy(x).cuda(), torch.full((m, n), float("nan"), device="cuda"), dtype, m, n, k)
                   for (w, x), n in zip(host, ns)]
        print(f"chain: open requests dtype={dtype} m={m} depth={depth}", flush=True)
        run_batch(backend, torch, entries, after_previous=None)
        # (a ring too short for the number asked for sends the entries to single launches: the same bits)
        if depth <= 2:
            assert backend.last_kernel_name().startswith("gq_mm8c_"), backend.last_kernel_name()
        outs.append([e[2].cpu().numpy() for e in entries])
    for depth, out in enumerate(outs[1:], 1):
        for i in range(len(ns)):
            assert np.array_equal(out[i].view(np.uint32), outs[0][i].view(np.uint32)), f"entry {i}, depth {depth}"
