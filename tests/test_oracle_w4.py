"""Pins oracle/w4.py: reference-held known-answer vectors, brute force, round trips, exactness."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import w4


def _kat_inputs(k, n):
    # AGQ/tests/test_q4.py:1071-1074,1097 and :1757-1764 -- draw order matters
    torch.manual_seed(42)
    qweight = torch.randint(-100, 100, size=(k // 8, n), dtype=torch.int32)
    scales = torch.zeros(k // 128, n, dtype=torch.float16) + 0.002
    qzeros = torch.zeros(k // 128, n // 8, dtype=torch.int32)
    inp = torch.rand(1, 1, k, dtype=torch.float16)
    return qweight, qzeros, scales, inp


@pytest.mark.parametrize("name", ["exllama_k1024_n1024", "cuda_old_half_k256_n256", "cuda_old_no_half_k256_n256"])
def test_reference_known_answer_vectors(golden_dir, name):
    kat = json.load(open(os.path.join(golden_dir, "q4_kat.json")))[name]
    k, n = kat["k"], kat["n"]
    qweight, qzeros, scales, inp = _kat_inputs(k, n)
    W = w4.dequantize(qweight, qzeros, scales, 128)
    out = w4.linear_fp32(inp[0], W)[0]
    ref = torch.tensor(kat["out"], dtype=torch.float32)
    # The stored vectors were produced by fp16 kernels with their own accumulation order:
    # agreement is to 2 fp16 ulp of the result (values are < 16, so 1 ulp <= 2^-7).
    ulp = torch.maximum(torch.tensor(2.0 ** -10), 2.0 ** (torch.floor(torch.log2(ref.abs())) - 10))
    assert ((out - ref).abs() <= 2 * ulp + 1e-6).all(), float((out - ref).abs().max())
    # and inside the reference's own tolerance for the exllama vector
    assert torch.allclose(out, ref, rtol=3e-5, atol=2e-2)
    # a dropped "+1" on the zero point shifts every output by 0.002*sum(inp) ~ 0.25..1.0: must fail
    wrong = out + 0.002 * inp.float().sum()
    assert not torch.allclose(wrong, ref, rtol=3e-5, atol=2e-2)


@pytest.mark.parametrize("K,N,g", [(128, 8, 128), (256, 16, 128), (256, 32, 64)])
def test_dequant_matches_bruteforce_and_literal(K, N, g):
    qw, qz, sc = w4.random_quantized(K, N, g, seed=K + N)
    a = w4.dequantize(qw, qz, sc, g)
    b = torch.from_numpy(w4.dequantize_bruteforce(qw, qz, sc, g))
    c = w4.dequantize_torch_literal(qw, qz, sc, g)
    assert a.dtype == torch.float16 and c.dtype == torch.float16
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    assert torch.equal(a.view(torch.int16), c.view(torch.int16))


def test_dequant_subnormal_and_zero_scales_survive():
    K, N, g = 128, 8, 128
    qw, qz, _ = w4.random_quantized(K, N, g, seed=3)
    sc = torch.tensor([[0.0, 6e-8, 1.2e-7, 3e-6, 5.9e-5, 6.2e-5, 1e-3, 65504.0 / 16]], dtype=torch.float16)
    a = w4.dequantize(qw, qz, sc, g)
    c = w4.dequantize_torch_literal(qw, qz, sc, g)
    assert torch.equal(a.view(torch.int16), c.view(torch.int16))
    assert (a[:, 0] == 0).all()
    sub = a[:, 1].float().abs()
    assert (sub[sub > 0] < 6.2e-5).all() and (sub > 0).any()  # subnormal products kept, not flushed
    q = w4.unpack_qweight(qw)[:, 1] - w4.unpack_qzeros(qz)[0, 1]
    assert torch.equal(a[:, 1].double(), (sc[0, 1].double() * q.double()).to(torch.float16).double())


def test_pack_unpack_round_trip():
    gen = torch.Generator().manual_seed(0)
    q = torch.randint(0, 16, (256, 24), generator=gen, dtype=torch.int32)
    assert torch.equal(w4.unpack_qweight(w4.pack_nibbles(q, 0)), q)
    z = torch.randint(0, 16, (2, 24), generator=gen, dtype=torch.int32)
    assert torch.equal(w4.unpack_qzeros(w4.pack_nibbles(z, 1)), z + 1)
    # nibble j of word r is element 8r+j (little nibble first): AGQ qlinear_cuda_old.py:122-130
    one = torch.zeros(8, 1, dtype=torch.int32)
    one[3, 0] = 0xA
    assert int(w4.pack_nibbles(one, 0)[0, 0]) == 0xA << 12


def test_pack_linear_quantises_back_to_grid():
    gen = torch.Generator().manual_seed(1)
    N, K, g = 16, 256, 128
    scales = (torch.rand(N, K // g, generator=gen) * 0.01 + 0.001).half().float()
    zeros = torch.randint(1, 17, (N, K // g), generator=gen)
    qtrue = torch.randint(0, 16, (N, K), generator=gen)
    gi = torch.arange(K) // g
    W = scales[:, gi] * (qtrue - zeros[:, gi]).float()
    qw, qz, s16 = w4.pack_linear(W, scales, zeros, g)
    assert torch.equal(w4.unpack_qweight(qw), qtrue.t().to(torch.int32))
    assert torch.equal(w4.unpack_qzeros(qz), zeros.t().to(torch.int32))
    Wd = w4.dequantize(qw, qz, s16, g)
    assert torch.allclose(Wd.float().t(), W, rtol=1e-3, atol=1e-6)


def test_dequant_act_order_g_idx_matches_bruteforce():
    """Per-row gather of scale and zero (``AGQ:qlinear_cuda.py:253-265``) against a scalar loop."""
    import numpy as np

    K, N, g = 256, 16, 128
    qw, qz, sc = w4.random_quantized(K, N, g, seed=3)
    g_idx = (torch.randperm(K, generator=torch.Generator().manual_seed(0)) // g).to(torch.int32)
    out = w4.dequantize(qw, qz, sc, g, g_idx)
    qwn, qzn = qw.numpy().astype(np.int64) & 0xFFFFFFFF, qz.numpy().astype(np.int64) & 0xFFFFFFFF
    scn = sc.numpy()
    for k in range(0, K, 7):
        gi = int(g_idx[k])
        for n in range(N):
            q = (int(qwn[k >> 3, n]) >> (4 * (k & 7))) & 15
            z = ((int(qzn[gi, n >> 3]) >> (4 * (n & 7))) & 15) + 1
            assert out[k, n].item() == float(np.float16(np.float32(scn[gi, n]) * np.float32(q - z)))
    assert torch.equal(w4.dequantize(qw, qz, sc, g, torch.arange(K) // g), w4.dequantize(qw, qz, sc, g))
