"""Writes tests/golden/q4_kat.json: the three known-answer output vectors that the
reference's own int4 kernel tests hold as literals
(``inference/compression/dependencies/AutoGPTQ/tests/test_q4.py``:
``TestsQ4Exllama.REFERENCE`` lines 21-1048, ``TestsQ4CUDA.REFERENCE_OLD_HALF`` 1213-1472,
``REFERENCE_OLD_NO_HALF`` 1474-1733), together with the recipe of their inputs
(lines 1071-1074, 1097, 1757-1764): ``torch.manual_seed(42)``; ``qweight =
randint(-100, 100, (K/8, N), int32)``; ``scales = 0.002`` (fp16); ``qzeros = 0``;
``inp = rand(1, 1, K, fp16)``, drawn in that order on the CPU generator.

The test file is read as text (it is never imported or executed); only numbers are kept.
Run in the build container:  python tests/golden/make_q4_kat.py
"""
import json
import os
import re

SRC = "/root/reference/inference/compression/dependencies/AutoGPTQ/tests/test_q4.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "q4_kat.json")


def grab(text: str, name: str):
    m = re.search(r"\b" + name + r" = torch\.Tensor\(\s*\[(.*?)\]\s*\)\.to\(torch\.float16\)", text, re.S)
    assert m, name
    return [float(t) for t in re.findall(r"-?\d+\.\d+(?:e-?\d+)?", m.group(1))]


def main():
    text = open(SRC).read()
    out = {
        "source": "AutoGPTQ tests/test_q4.py (vendored in the reference), literals only",
        "recipe": {"seed": 42, "qweight": "randint(-100,100,(K/8,N),int32)", "scales": 0.002, "qzeros": 0,
                   "inp": "rand(1,1,K,float16)", "group_size": 128},
        "exllama_k1024_n1024": {"k": 1024, "n": 1024, "rtol": 3e-5, "atol": 2e-2, "out": grab(text, "REFERENCE")},
        "cuda_old_half_k256_n256": {"k": 256, "n": 256, "out": grab(text, "REFERENCE_OLD_HALF")},
        "cuda_old_no_half_k256_n256": {"k": 256, "n": 256, "out": grab(text, "REFERENCE_OLD_NO_HALF")},
    }
    assert len(out["exllama_k1024_n1024"]["out"]) == 1024
    assert len(out["cuda_old_half_k256_n256"]["out"]) == 256
    assert len(out["cuda_old_no_half_k256_n256"]["out"]) == 256
    with open(OUT, "w") as f:
        json.dump(out, f)
    print("wrote", OUT)


if __name__ == "__main__":
    main()
