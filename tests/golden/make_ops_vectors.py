"""Writes tests/golden/ops_vectors.npz: inputs and outputs of the reference's own torch implementations of
merge_attn_states, attention_update_torch and gather_and_maybe_dequant_cache (src/omni_npu/attention/ops.py), for the
edge-case conventions that mathematics does not fix (+inf log-sum-exps read as -inf, rows with no weight at all).

Run in the build container only (the reference tree is not present anywhere else):
    python tests/golden/make_ops_vectors.py
The reference file imports nothing but `typing` and `torch`; it is loaded by path, nothing of it is copied or shipped.
"""
import importlib.util
import os

import numpy as np
import torch

REF = "/root/reference/src/omni_npu/attention/ops.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ops_vectors.npz")


def load_reference():
    spec = importlib.util.spec_from_file_location("reference_attention_ops", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def main():
    ref = load_reference()
    g = torch.Generator().manual_seed(20240607)
    inf = float("inf")
    vec = {}

    # --- merge_attn_states: (T, N, D) bf16 outputs, (T, N, 1) fp32 log-sum-exps; rows exercise every convention ---
    t, n, d = 8, 3, 16
    po = torch.randn(t, n, d, generator=g).bfloat16()
    so = torch.randn(t, n, d, generator=g).bfloat16()
    pl = torch.randn(t, n, 1, generator=g) * 3
    sl = torch.randn(t, n, 1, generator=g) * 3
    pl[1], sl[2] = inf, inf                      # +inf reads as -inf: the other side is returned
    pl[3], sl[3] = -inf, 1.5                     # nothing in the prefix
    pl[4], sl[4] = -inf, -inf                    # nothing at all: zeros and -inf
    pl[5], sl[5] = inf, inf                      # both +inf: zeros and -inf
    pl[6], sl[6] = 40.0, -40.0                   # one side dominates completely
    out = torch.full((t, n, d), float("nan"), dtype=torch.float32)
    out_lse = torch.full((t, n, 1), float("nan"), dtype=torch.float32)
    ref.merge_attn_states(out, po, pl, so, sl, out_lse)
    vec.update(merge_prefix_out=po.float().numpy(), merge_suffix_out=so.float().numpy(), merge_prefix_lse=pl.numpy(),
               merge_suffix_lse=sl.numpy(), merge_out=out.numpy(), merge_out_lse=out_lse.numpy())

    # --- attention_update_torch: n partials [n, T, D] fp32 (values exactly representable in fp16), lses [n, T] ---
    npart, t2, d2 = 5, 7, 16
    outs = torch.randn(npart, t2, d2, generator=g).half().float()
    lses = torch.randn(npart, t2, generator=g) * 4
    lses[:, 1] = -inf                            # a row without any weight
    lses[2, 2] = inf                             # +inf reads as -inf
    lses[:, 3] = inf                             # every partial +inf
    lses[0, 4], lses[1:, 4] = 3.0, -inf          # a single live partial
    lses[:, 5] = torch.tensor([60.0, -60.0, 0.0, 59.0, -inf])
    upd_out, upd_lse = ref.attention_update_torch(outs.clone(), lses.clone())
    vec.update(update_outs=outs.numpy(), update_lses=lses.numpy(), update_out=upd_out.numpy(), update_lse=upd_lse.numpy())

    # --- gather_and_maybe_dequant_cache: paged rows -> contiguous workspace (structured values: pure data movement) ---
    pages, page, dn, dr = 5, 128, 512, 64
    idx = torch.arange(pages * page).view(pages, page, 1)
    nope = ((idx * 7 + torch.arange(dn).view(1, 1, dn) * 3) % 509 - 254).to(torch.bfloat16)
    rope = ((idx * 5 + torch.arange(dr).view(1, 1, dr) * 11) % 251 - 125).to(torch.bfloat16)
    block_table = torch.tensor([[3, 0, 4], [1, 2, 0], [4, 1, 3]], dtype=torch.int32)
    seq_starts = torch.tensor([0, 100, 130], dtype=torch.int32)
    lens = [200, 77, 0]                          # crosses a page border, starts inside a page, empty
    cu = torch.tensor([0, 200, 277, 277], dtype=torch.int32)
    dst = torch.full((277, dn + dr), -7.0, dtype=torch.bfloat16)
    ref.gather_and_maybe_dequant_cache((nope, rope), dst, block_table.long(), cu, 3, "auto", torch.tensor(1.0), seq_starts)
    vec.update(gather_block_table=block_table.numpy(), gather_seq_starts=seq_starts.numpy(), gather_cu=cu.numpy(),
               gather_dst=dst.float().numpy(), gather_shape=np.array([pages, page, dn, dr], dtype=np.int64))
    np.savez_compressed(OUT, **vec)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
