"""Writes tests/golden/hf_olmo2_kat.npz: logits of ``transformers``' own ``Olmo2ForCausalLM`` (MHA and GQA,
perturbed norm weights) and ``OlmoForCausalLM`` (non-parametric LayerNorm, pre-norm, with and without
``clip_qkv``) on the seeded weights and inputs of ``hf_kat_recipe.py``, with and without a left-padding mask.

Run in the build container (CPU, fp32):  python tests/golden/make_hf_olmo2_kat.py
Nothing of the reference is imported or run; ``transformers`` is the installed third-party package.
Only positions whose token is real are stored as checked values (padding rows are kept too, flagged by the mask).
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from tests.golden import hf_kat_recipe as R  # noqa: E402

OUT = os.path.join(HERE, "hf_olmo2_kat.npz")


def main():
    import transformers

    torch.manual_seed(0)
    out = {"versions": np.array([f"transformers {transformers.__version__}", f"torch {torch.__version__}"])}
    for name, case in R.CASES.items():
        seed = R.seed_of(name)
        sd = R.hf_state_dict(case, seed)
        m = R.hf_model(case, sd)
        ids, mask = R.inputs(case, seed)
        with torch.no_grad():
            plain = m(input_ids=ids).logits
            padded = m(input_ids=ids, attention_mask=mask).logits
        out[name + ".logits"] = plain.numpy().astype(np.float32)
        out[name + ".logits_left_padded"] = padded.numpy().astype(np.float32)
        print(name, tuple(plain.shape), float(plain.abs().max()))
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
