"""From a GGUF file to tokens on the GPU: the reader's tensors uploaded as stored and run through
the quantized embedding lookup, a feed-forward block, the lm_head matvec and the greedy token
choice, against the oracle on the same bytes."""
import os

import numpy as np
import pytest

from gllm_amd.gguf import GgufFile
from gllm_amd.synth import random_weight
from tests import gguf_writer as W

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14


@pytest.fixture(scope="module")
def hip():
    from gllm_amd.backend import HipBackend
    return HipBackend(0)


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def test_gguf_to_tokens(hip, torch, oracle, tmp_path):
    vocab, hidden, ffn = 300, 512, 768
    print("gguf to tokens", flush=True)
    host = {
        "token_embd.weight": (Q4_K, vocab, hidden, random_weight(Q4_K, vocab, hidden, seed=1)),
        "blk.0.ffn_gate.weight": (Q5_K, ffn, hidden, random_weight(Q5_K, ffn, hidden, seed=2)),
        "blk.0.ffn_up.weight": (Q5_K, ffn, hidden, random_weight(Q5_K, ffn, hidden, seed=3)),
        "blk.0.ffn_down.weight": (Q6_K, hidden, ffn, random_weight(Q6_K, hidden, ffn, seed=4)),
        "output.weight": (Q8_0, vocab, hidden, random_weight(Q8_0, vocab, hidden, seed=5)),
    }
    meta = [("general.architecture", W.STR, "llama"), ("llama.embedding_length", W.U32, hidden),
            ("llama.feed_forward_length", W.U32, ffn), ("general.alignment", W.U32, 64)]
    tensors = [(name, [k, n], dt, np.asarray(w).tobytes()) for name, (dt, n, k, w) in host.items()]
    path = os.path.join(tmp_path, "tiny.gguf")
    with open(path, "wb") as f:
        f.write(W.build(meta, tensors))

    g = GgufFile(path)
    assert g.meta("llama.embedding_length") == hidden and g.alignment == 64
    dev = {}
    for name, (dt, n, k, w) in host.items():
        t = g.tensor(name)
        assert t.shape == (n, k) and t.ggml_dtype == dt and t.nbytes == np.asarray(w).nbytes
        buf = torch.empty(t.nbytes + 64, dtype=torch.uint8, device="cuda")
        buf[t.nbytes:] = 0xAB
        g.upload(hip, name, buf[:t.nbytes])
        torch.cuda.synchronize()
        assert bytes(buf[:t.nbytes].cpu().numpy()) == np.asarray(w).tobytes()
        assert bool(torch.all(buf[t.nbytes:] == 0xAB)), "upload wrote past the tensor"
        dev[name] = buf[:t.nbytes]
    with pytest.raises(Exception):
        g.upload(hip, "output.weight", dev["output.weight"][:100])  # destination too small

    ids = np.array([7, 299, 0, 123], np.uint32)
    m = len(ids)
    idd = torch.from_numpy(ids.view(np.int32)).cuda()
    x = torch.empty(m, hidden, device="cuda")
    h = torch.empty(m, hidden, device="cuda")
    logits = torch.empty(m, vocab, device="cuda")
    tok = torch.zeros(m, dtype=torch.int32, device="cuda")
    hip.quant_gather(dev["token_embd.weight"], Q4_K, vocab, hidden, idd, x)
    hip.ffn_swiglu(dev["blk.0.ffn_gate.weight"], dev["blk.0.ffn_up.weight"], Q5_K, dev["blk.0.ffn_down.weight"], Q6_K,
                   x, h, m, hidden, ffn)
    hip.quantized_matmul(dev["output.weight"], h, logits, Q8_0, m, vocab, hidden)
    hip.argmax(logits, tok)
    torch.cuda.synchronize()

    ex = oracle.quant_gather(host["token_embd.weight"][3], Q4_K, vocab, hidden, ids)
    assert np.array_equal(x.cpu().numpy().view(np.uint32), ex.view(np.uint32))
    eh = oracle.ffn_swiglu(host["blk.0.ffn_gate.weight"][3], host["blk.0.ffn_up.weight"][3], Q5_K,
                           host["blk.0.ffn_down.weight"][3], Q6_K, ex, m, hidden, ffn, acc=oracle.ACC_F64, threads=4)
    el = oracle.quantized_matmul(host["output.weight"][3], eh, Q8_0, m, vocab, hidden, acc=oracle.ACC_F64, threads=4)
    got = logits.cpu().numpy()
    rel = np.linalg.norm(got - el) / np.linalg.norm(el)
    assert rel <= 1e-4, rel
    assert tok.cpu().numpy().tolist() == [oracle.argmax_token(got[r]) for r in range(m)]
    for r in range(m):
        assert el[r, int(tok[r])] >= el[r].max() - 2e-3 * np.abs(el[r]).max()


def test_mixed_quant_layers_from_the_layer_table(hip, torch, oracle, tmp_path):
    """A Q4_K_M-style file (ffn_down Q6_K in layers 0 and 3, Q4_K in 1 and 2): the host walks the
    layer table and calls the same entry point with each matrix's own dtype."""
    from tests.test_gguf_reader import k_m_style_file
    print("mixed-quant layers", flush=True)
    image, host = k_m_style_file()
    path = os.path.join(tmp_path, "km.gguf")
    with open(path, "wb") as f:
        f.write(image)
    g = GgufFile(path)
    assert [layers for _, layers in g.mixed_quant_groups()] == [[1, 2], [0, 3]]
    hidden, ffn, m = 256, 512, 2
    x = np.random.default_rng(0).standard_normal((m, hidden)).astype(np.float32)
    xd, want = torch.from_numpy(x).cuda(), x
    for layer, projs in g.layer_table().items():
        dev = {}
        for proj, t in projs.items():
            dev[proj] = torch.empty(t.nbytes, dtype=torch.uint8, device="cuda")
            g.upload(hip, t.name, dev[proj])
        out = torch.empty(m, hidden, device="cuda")
        hip.ffn_swiglu(dev["ffn_gate"], dev["ffn_up"], projs["ffn_gate"].ggml_dtype, dev["ffn_down"],
                       projs["ffn_down"].ggml_dtype, xd, out, m, hidden, ffn)
        torch.cuda.synchronize()
        names = [f"blk.{layer}.{p}.weight" for p in ("ffn_gate", "ffn_up", "ffn_down")]
        want = oracle.ffn_swiglu(host[names[0]][3], host[names[1]][3], host[names[0]][0], host[names[2]][3],
                                 host[names[2]][0], want, m, hidden, ffn, acc=oracle.ACC_F64, threads=4)
        got = out.cpu().numpy()
        rel = np.linalg.norm(got - want) / np.linalg.norm(want)
        assert rel <= 1e-4, (layer, rel)
        # the next layer continues from the GPU's own output, normalised so that magnitudes stay put
        scale = float(np.abs(got).max())
        xd, want = out / scale, (got / np.float32(scale)).astype(np.float32)
