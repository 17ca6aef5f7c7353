"""GPU parity of the greedy token choice (gllmq_argmax through the C ABI) against the oracle's
argmax_token, which is pinned by the reference's unit-test vectors: index-exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

NAN = float("nan")
NONE = 0xFFFFFFFF


@pytest.fixture(scope="module")
def hip():
    from gllm_amd.backend import HipBackend
    return HipBackend(0)


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def gpu_argmax(hip, torch, rows):
    """rows: list of equally long vectors; returns (tokens, values) with NaN poison behind the logits."""
    a = np.asarray(rows, np.float32).reshape(len(rows), -1)
    m, n = a.shape
    buf = torch.full((m * n + 4096,), NAN, dtype=torch.float32, device="cuda")
    buf[:m * n] = torch.from_numpy(a.reshape(-1)).cuda()
    tok = torch.full((m + 8,), 12345, dtype=torch.int32, device="cuda")
    val = torch.full((m + 8,), 7.0, dtype=torch.float32, device="cuda")
    hip.argmax(buf[:m * n].view(m, n), tok[:m], val[:m])
    torch.cuda.synchronize()
    assert bool(torch.all(tok[m:] == 12345)) and bool(torch.all(val[m:] == 7.0)), "write past the outputs"
    return tok[:m].cpu().numpy().view(np.uint32), val[:m].cpu().numpy()


def check(hip, torch, oracle, rows, what):
    tok, val = gpu_argmax(hip, torch, rows)
    for r, row in enumerate(np.asarray(rows, np.float32).reshape(len(rows), -1)):
        want = oracle.argmax_token(row)
        if want is None:
            assert tok[r] == NONE and np.isnan(val[r]), (what, r, tok[r])
        else:
            assert tok[r] == want, (what, r, tok[r], want)
            assert val[r] == row[want] or (val[r] == 0.0 and row[want] == 0.0), (what, r, val[r], row[want])


def test_reference_vectors(hip, torch, oracle):
    print("argmax reference vectors", flush=True)
    for v in ([0.1, 0.2, 0.5, 0.9, 0.3], [42.0], [1.0, 5.0, 5.0, 2.0], [3.0, 3.0, 3.0], [0.1, 0.2, 0.3, 0.4, 99.0],
              [-10.0, -5.0, -20.0], [NAN, 1.0], [NAN, NAN, NAN], [0.0, -0.0], [-0.0, 0.0], [float("-inf"), NAN],
              [float("inf"), 1.0, float("inf")], [NAN, -1.0, NAN, -1.0, NAN]):
        check(hip, torch, oracle, [v], str(v))
    big = np.zeros(10000, np.float32)
    big[7777] = 1.0
    check(hip, torch, oracle, [big], "large slice")


@pytest.mark.parametrize("n", [1, 63, 256, 4096, 4097, 32000, 151936])
def test_random_rows_with_ties_and_nans(hip, torch, oracle, n):
    print(f"argmax random n={n}", flush=True)
    rng = np.random.default_rng(n)
    rows = []
    for r in range(5):
        v = np.round(rng.standard_normal(n).astype(np.float32) * 4) / 4  # quarter steps: many exact ties
        if r >= 2:
            v[rng.integers(0, n, max(1, n // 10))] = NAN
        if r == 4:
            v[:] = NAN
            v[rng.integers(0, n)] = -3.0
        rows.append(v)
    check(hip, torch, oracle, rows, f"n={n}")


def test_more_rows_than_one_launch_covers_and_row_stride(hip, torch, oracle):
    print("argmax 70 rows with a stride", flush=True)
    rng = np.random.default_rng(1)
    m, n, ld = 70, 5000, 5008
    a = rng.standard_normal((m, ld)).astype(np.float32)
    a[:, n:] = 1e9  # entries behind the row's end must not win
    buf = torch.from_numpy(a).cuda()
    tok = torch.zeros(m, dtype=torch.int32, device="cuda")
    hip.argmax(buf[:, :n], tok)
    torch.cuda.synchronize()
    got = tok.cpu().numpy()
    want = np.array([oracle.argmax_token(a[r, :n]) for r in range(m)])
    assert np.array_equal(got, want)


def test_lm_head_then_argmax(hip, torch, oracle):
    """The end of a decode step: Q6_K lm_head matvec over a 32000-token vocabulary, then the token."""
    from gllm_amd.synth import random_activations, random_weight
    print("lm_head + argmax", flush=True)
    n, k = 32000, 2048
    w, x = random_weight(14, n, k, seed=8), random_activations(2, k, seed=9)
    wd = torch.from_numpy(np.asarray(w).view(np.uint8)).cuda()
    xd = torch.from_numpy(x).cuda()
    y = torch.empty(2, n, device="cuda")
    tok = torch.zeros(2, dtype=torch.int32, device="cuda")
    hip.quantized_matmul(wd, xd, y, 14, 2, n, k)
    hip.argmax(y, tok)
    torch.cuda.synchronize()
    yh = y.cpu().numpy()
    assert [oracle.argmax_token(yh[r]) for r in range(2)] == tok.cpu().numpy().tolist()
    # and the token is the oracle's own choice unless two of its logits are closer than the matmul tolerance
    want = oracle.quantized_matmul(w, x, 14, 2, n, k, acc=oracle.ACC_F64, threads=8)
    for r in range(2):
        t = int(tok[r])
        assert want[r, t] >= want[r].max() - 2e-3 * np.abs(want[r]).max()


@pytest.mark.parametrize("dt,n,k", [(14, 32000, 2048), (14, 128256, 4096), (14, 1000, 8192), (14, 37, 256), (8, 5000, 1024),
                                     (8, 777, 12288), (12, 32000, 2048), (13, 3000, 1024), (14, 300, 16640)])
def test_lm_head_and_token_in_one_call(hip, torch, oracle, dt, n, k):
    """gllmq_lm_head_argmax against the two calls it stands for: the same logits and the same token bit
    for bit, with and without a logits buffer (Q6_K and Q8_0 within one launch of K never write
    them; other matrices need the buffer), and the token against the oracle's choice on its own logits."""
    from gllm_amd.backend import BackendError
    from gllm_amd.synth import random_activations, random_weight
    print(f"lm_head_argmax dtype={dt} n={n} k={k}", flush=True)
    w, x = random_weight(dt, n, k, seed=n), random_activations(1, k, seed=k)
    wd = torch.from_numpy(np.asarray(w).view(np.uint8).reshape(-1)).cuda()
    xd = torch.from_numpy(x).cuda()
    y = torch.empty(1, n, device="cuda")
    tok = torch.zeros(1, dtype=torch.int32, device="cuda")
    val = torch.zeros(1, device="cuda")
    hip.quantized_matmul(wd, xd, y, dt, 1, n, k)
    hip.argmax(y, tok, val)
    torch.cuda.synchronize()
    y2 = torch.full((n + 64,), NAN, device="cuda")
    tok2 = torch.full((4,), 12345, dtype=torch.int32, device="cuda")
    val2 = torch.full((4,), 7.0, device="cuda")
    hip.lm_head_argmax(wd, xd, dt, n, k, tok2[:1], logits=y2[:n], value=val2[:1])
    torch.cuda.synchronize()
    assert torch.equal(y2[:n], y[0]) and bool(torch.all(torch.isnan(y2[n:])))
    assert int(tok2[0]) == int(tok[0]) and float(val2[0]) == float(val[0])
    assert tok2[1:].tolist() == [12345] * 3 and val2[1:].tolist() == [7.0] * 3
    tok3 = torch.full((1,), 777, dtype=torch.int32, device="cuda")
    if dt in (14, 8) and k <= 16384:
        hip.lm_head_argmax(wd, xd, dt, n, k, tok3)
        torch.cuda.synchronize()
        assert int(tok3[0]) == int(tok[0])
    else:
        with pytest.raises(BackendError):
            hip.lm_head_argmax(wd, xd, dt, n, k, tok3)
    yh = y.cpu().numpy()[0]
    assert oracle.argmax_token(yh) == int(tok[0])
    want = oracle.quantized_matmul(w, x, dt, 1, n, k, acc=oracle.ACC_F64, threads=8)[0]
    assert want[int(tok[0])] >= want.max() - 2e-3 * np.abs(want).max()


def test_lm_head_token_with_ties_and_nan(hip, torch, oracle):
    """Rows of equal weights give equal logits (the LAST of them is the token), and a NaN activation
    leaves no candidate at all."""
    from gllm_amd.synth import random_activations, random_weight
    print("lm_head_argmax ties and NaN", flush=True)
    dt, n, k = 14, 4000, 1024
    w = np.asarray(random_weight(dt, n, k, seed=1)).view(np.uint8).reshape(n, -1).copy()
    x = random_activations(1, k, seed=2)
    first = oracle.quantized_matmul(w.reshape(-1), x, dt, 1, n, k, acc=oracle.ACC_F64, threads=4)[0]
    top = int(np.argmax(first))
    for r in (5, 1999, 3998):  # copies of the winning row, in different workgroups
        w[r] = w[top]
    wd = torch.from_numpy(w.reshape(-1)).cuda()
    tok = torch.zeros(1, dtype=torch.int32, device="cuda")
    val = torch.zeros(1, device="cuda")
    hip.lm_head_argmax(wd, torch.from_numpy(x).cuda(), dt, n, k, tok, value=val)
    torch.cuda.synchronize()
    assert int(tok[0]) == max(top, 3998)
    xn = x.copy()
    xn[0, 100] = NAN
    hip.lm_head_argmax(wd, torch.from_numpy(xn).cuda(), dt, n, k, tok, value=val)
    torch.cuda.synchronize()
    y = torch.empty(1, n, device="cuda")
    hip.quantized_matmul(wd, torch.from_numpy(xn).cuda(), y, dt, 1, n, k)
    want = oracle.argmax_token(y.cpu().numpy()[0])
    assert (int(tok[0]) & 0xFFFFFFFF) == (NONE if want is None else want)


def test_argument_errors(hip, torch):
    from gllm_amd.backend import BackendError
    print("argmax errors", flush=True)
    tok = torch.full((2,), 5, dtype=torch.int32, device="cuda")
    hip.argmax(torch.zeros(0, 8, device="cuda"), tok)            # no rows: nothing written
    hip.argmax(torch.zeros(2, 0, device="cuda"), tok)            # empty rows: no token
    torch.cuda.synchronize()
    assert tok.cpu().numpy().view(np.uint32).tolist() == [NONE, NONE]
    with pytest.raises(BackendError):
        hip.argmax(torch.zeros(2, 8, device="cuda", dtype=torch.float16), tok)
