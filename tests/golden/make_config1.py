"""Writes tests/golden/config1_decode.npz: the oracle's absorbed-MLA decode on the CPU-plumbing configuration
(16 heads, batch 4, lens uniform in [128,1024], page 128, shuffled block tables, N(0,1) bf16, scale 1/sqrt(192),
seed 0).  The reference holds no stored vectors for this path (its numeric tests draw from an NPU generator), so
the fixture records this repository's oracle; run from the repository root:  python tests/golden/make_config1.py"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import mla_oracle as O  # noqa: E402

c = O.make_decode_case(4, 16, 128, 1024, seed=0)
out, lse = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], c["scale"],
                             return_lse=True)
np.savez_compressed(os.path.join(ROOT, "tests", "golden", "config1_decode.npz"), seq_lens=c["seq_lens"].numpy(),
                    block_table=c["block_table"].numpy(), out=out.numpy().astype(np.float16), lse=lse.numpy())
print("written", out.shape)
