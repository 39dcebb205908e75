"""GPU parity of the decode tail (final RMSNorm + bf16 lm_head GEMV + argmax) against the oracle."""
import numpy as np
import pytest
import torch

from helpers import assert_bf16_close
from oracle import decode as odec
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def dev(a):
    a = np.ascontiguousarray(a)
    return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)


def bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.fixture(scope="module")
def ops():
    from air_hip import ops
    return ops


def _inputs(V, E, seed):
    rng = np.random.default_rng(seed)
    x = f32_to_bf16_bits((rng.standard_normal(E) * 2.0).astype(np.float32))
    nw = f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32))
    W = f32_to_bf16_bits((rng.standard_normal((V, E)) * 0.05).astype(np.float32))
    return x, nw, W


def _check(ops, x, nw, W, eps=1e-5):
    V, E = W.shape
    print(f"lm_head V={V} E={E} norm={nw is not None}", flush=True)
    logits, best = ops.lm_head(dev(x), dev(W), norm_weight=None if nw is None else dev(nw), eps=eps)
    torch.cuda.synchronize()
    got = bits(logits)
    # the kernel's argmax is exactly np.argmax of the logits it returned
    assert int(best.item()) == int(np.argmax(bf16_bits_to_f32(got).astype(np.float32)))
    # logits against the float64 product of the oracle's normalised vector: one bf16 ulp plus the
    # effect of a one-ulp flip of a normalised element (the kernel sums x^2 in another order)
    normed = np.asarray(x) if nw is None else odec.final_rms_norm(x, nw, eps)
    nf = bf16_bits_to_f32(normed).astype(np.float64)
    wf = bf16_bits_to_f32(W).astype(np.float64)
    want = wf @ nf
    slack = 0.0 if nw is None else 2.0**-8 * float(np.sqrt((wf * wf).sum(axis=1).max()) * np.abs(nf).max())
    assert_bf16_close(got, want, ulps=1.0, atol=slack + 1e-6, what=f"lm_head V={V} E={E}")
    want_bits, want_best = odec.lm_head_reference(x, nw, W, eps)
    top2 = np.sort(want)[-2:]
    if V == 1 or top2[1] - top2[0] > 4 * 2.0**-8 * abs(top2[1]) + 2 * slack:
        assert int(best.item()) == want_best
    return got


@pytest.mark.parametrize("V,E", [(1000, 512), (4096, 1024), (333, 1536), (2048, 2048), (777, 3072), (1024, 4096),
                                 (500, 5120), (256, 8192), (64, 256), (100, 8), (300, 2560), (129, 6152)])
def test_lm_head_shapes(ops, V, E):
    x, nw, W = _inputs(V, E, seed=V + E)
    _check(ops, x, nw, W)
    _check(ops, x, None, W)


@pytest.mark.parametrize("V", [1, 15, 16, 17, 63, 65, 1025])
def test_lm_head_ragged_vocabulary(ops, V):
    x, nw, W = _inputs(V, 2048, seed=V)
    _check(ops, x, nw, W)


def test_lm_head_exact_cases(ops):
    """One-hot rows return elements of the input bit for bit; tied rows give the first index."""
    V, E = 640, 2048
    x, nw, W = _inputs(V, E, seed=5)
    idx = (7 * np.arange(V)) % E
    onehot = np.zeros((V, E), np.uint16)
    onehot[np.arange(V), idx] = 0x3F80
    logits, best = ops.lm_head(dev(x), dev(onehot), norm_weight=None)
    torch.cuda.synchronize()
    assert np.array_equal(bits(logits), x[idx])
    assert int(best.item()) == odec.lm_head_reference(x, None, onehot)[1]
    # three equal rows that hold the maximum: x itself as a row gives sum(x^2), the largest product for its norm
    W[300] = W[45] = W[611] = x
    _, best = ops.lm_head(dev(x), dev(W), norm_weight=None)
    assert int(best.item()) == 45
    # all logits zero, of either sign: index 0
    z = np.zeros((V, E), np.uint16)
    z[0, 0] = 0x8000
    lz, best = ops.lm_head(dev(x), dev(z), norm_weight=None)
    assert int(best.item()) == 0 and np.all((bits(lz) & 0x7FFF) == 0)


def test_lm_head_llama32_1b_size(ops):
    """The reference's shape: vocabulary 128256, emb_dim 2048 (525 MB of weights)."""
    V, E = 128256, 2048
    g = torch.Generator(device="cuda").manual_seed(11)
    W = (torch.randn((V, E), device="cuda", generator=g) * 0.05).to(torch.bfloat16)
    x = (torch.randn((E,), device="cuda", generator=g) * 2.0).to(torch.bfloat16)
    nw = (torch.randn((E,), device="cuda", generator=g) * 0.1 + 1.0).to(torch.bfloat16)
    print("lm_head 128256 x 2048", flush=True)
    logits, best = ops.lm_head(x, W, norm_weight=nw)
    torch.cuda.synchronize()
    got = bits(logits)
    assert int(best.item()) == int(np.argmax(bf16_bits_to_f32(got).astype(np.float32)))
    normed = odec.final_rms_norm(bits(x), bits(nw))
    nf = torch.from_numpy(bf16_bits_to_f32(normed)).double()
    want = (W.cpu().double() @ nf).numpy()
    slack = 2.0**-8 * float(W.float().norm(dim=1).max()) * float(nf.abs().max())
    assert_bf16_close(got, want, ulps=1.0, atol=slack, what="lm_head at the 1B model's size")
    # repeatable bit for bit
    again, best2 = ops.lm_head(x, W, norm_weight=nw)
    assert torch.equal(again.view(torch.int16), logits.view(torch.int16)) and int(best2.item()) == int(best.item())


def test_lm_head_rejects_bad_arguments(ops):
    from air_hip import _lib
    lib = _lib.load_library()
    buf = torch.zeros(4096, dtype=torch.bfloat16, device="cuda")
    ws = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    p = buf.data_ptr()
    assert lib.lm_head_gemv_bf16(p, None, 0.0, p, p, None, 4, 8200, ws.data_ptr(), ws.numel(), None) == -2   # E above 8192
    assert lib.lm_head_gemv_bf16(None, None, 0.0, p, p, None, 4, 512, ws.data_ptr(), ws.numel(), None) == -1
    assert lib.lm_head_gemv_bf16(p, None, 0.0, p, p, None, 4, 512, ws.data_ptr(), 0, None) == -5
    assert lib.lm_head_gemv_bf16(p + 2, None, 0.0, p, p, None, 4, 512, ws.data_ptr(), ws.numel(), None) == -4
