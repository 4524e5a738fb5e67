"""The oracle's merges and gather against vectors written by the reference's own torch implementations
(tests/golden/ops_vectors.npz, made by tests/golden/make_ops_vectors.py from src/omni_npu/attention/ops.py), and the
closed form of the per-token fp8 quantiser."""
import os

import numpy as np
import torch

from oracle import mla_oracle as O

VEC = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ops_vectors.npz"))


def t(name, dtype=None):
    x = torch.from_numpy(VEC[name])
    return x.to(dtype) if dtype is not None else x


def gather_caches():
    """The structured caches of the gather vector (pure data movement: the values name their own row)."""
    pages, page, dn, dr = (int(v) for v in VEC["gather_shape"])
    idx = torch.arange(pages * page).view(pages, page, 1)
    nope = ((idx * 7 + torch.arange(dn).view(1, 1, dn) * 3) % 509 - 254).to(torch.bfloat16)
    rope = ((idx * 5 + torch.arange(dr).view(1, 1, dr) * 11) % 251 - 125).to(torch.bfloat16)
    return nope, rope


def same_with_inf(a, b, atol):
    """Equal where infinite (same sign), close where finite."""
    fin = torch.isfinite(b)
    return torch.equal(torch.isfinite(a), fin) and torch.equal(a[~fin], b[~fin]) and \
        torch.allclose(a[fin], b[fin], atol=atol, rtol=1e-6)


def test_merge_attn_states_matches_the_reference_vectors():
    out, lse = O.merge_attn_states(t("merge_prefix_out", torch.bfloat16), t("merge_prefix_lse"), t("merge_suffix_out", torch.bfloat16),
                                   t("merge_suffix_lse"))
    assert torch.allclose(out, t("merge_out"), atol=1e-6, rtol=1e-6)
    assert same_with_inf(lse, t("merge_out_lse"), 1e-6)
    # the vector really holds the conventions: rows 4 and 5 (nothing on either side / +inf on both) are zeros and -inf
    ref = t("merge_out")
    assert (ref[4] == 0).all() and (ref[5] == 0).all() and (t("merge_out_lse")[4:6] == float("-inf")).all()
    assert torch.equal(ref[1], t("merge_suffix_out")[1]) and torch.equal(ref[2], t("merge_prefix_out")[2])


def test_attention_update_matches_the_reference_vectors():
    out, lse = O.attention_update(t("update_outs"), t("update_lses"))
    assert torch.allclose(out, t("update_out"), atol=1e-6, rtol=1e-6)
    assert same_with_inf(lse, t("update_lse"), 1e-6)
    ref, ref_lse = t("update_out"), t("update_lse")
    assert (ref[1] == 0).all() and ref_lse[1] == float("-inf") and (ref[3] == 0).all() and ref_lse[3] == float("-inf")
    assert torch.equal(ref[4], t("update_outs")[0, 4]) and ref_lse[4] == 3.0          # the single live partial comes through


def test_attention_update_equals_a_fold_of_two_way_merges():
    """Associativity ties the N-way vector to the two-way one."""
    outs, lses = t("update_outs"), t("update_lses")
    acc, acc_l = outs[0].unsqueeze(1), lses[0].view(-1, 1, 1)
    for i in range(1, outs.shape[0]):
        acc, acc_l = O.merge_attn_states(acc, acc_l, outs[i].unsqueeze(1), lses[i].view(-1, 1, 1))
    z = torch.zeros_like(acc)
    acc, acc_l = O.merge_attn_states(acc, acc_l, z, torch.full_like(acc_l, float("-inf")))     # (normalises a lone +inf)
    assert torch.allclose(acc.squeeze(1), t("update_out"), atol=1e-5, rtol=1e-5)
    assert same_with_inf(acc_l.view(-1), t("update_lse"), 1e-5)


def test_gather_paged_matches_the_reference_vector():
    nope, rope = gather_caches()
    cu = t("gather_cu")
    dst = torch.full((int(cu[-1]), 576), -7.0, dtype=torch.bfloat16)
    O.gather_paged(nope, rope, dst, t("gather_block_table"), cu, 3, t("gather_seq_starts"))
    assert torch.equal(dst.float(), t("gather_dst"))


def test_fp8_token_quant_closed_form():
    g = torch.Generator().manual_seed(11)
    x = torch.randn(9, 128, generator=g) * 5
    x[0] = 0                                                     # an all-zero row: scale 1, zeros
    x[1, 7] = -1234.5                                            # the extreme is negative
    q, s = O.fp8_quant_token(x)
    assert q.dtype == torch.float8_e4m3fn and s.shape == (9,) and s.dtype == torch.float32
    amax = x.abs().amax(-1)
    assert s[0] == 1.0 and (q[0].float() == 0).all()
    assert torch.equal(s[1:], amax[1:] / 448.0)                  # scale = amax / 448 exactly (one fp32 division)
    # the extreme element lands on +-448, nothing exceeds it
    assert q[1, 7].float() == -448.0 and q.float().abs().max() == 448.0
    for r in range(1, 9):
        assert q[r].float().abs().max() == 448.0
    # round to nearest: the error of x / scale is at most half an e4m3 ulp of its binade (3 mantissa bits; 2^-9 below 2^-6)
    y = x[1:] / s[1:, None]
    err = (q[1:].float() - y).abs()
    ulp = torch.where(y.abs() >= 2.0 ** -6, 2.0 ** (torch.floor(torch.log2(y.abs().clamp_min(2.0 ** -6))) - 3), torch.tensor(2.0 ** -9))
    assert (err <= ulp / 2 + 1e-7).all()
    # values on the e4m3 grid with amax = 448 survive bit for bit (scale 1); ties go to the even mantissa
    grid = torch.tensor([448.0, -240.0, 1.5, 0.015625, 2.0 ** -9, 0.0] + [0.0] * 122)
    q2, s2 = O.fp8_quant_token(grid.view(1, 128))
    assert s2.item() == 1.0 and torch.equal(q2.float().view(-1), grid)
    ties = torch.tensor([448.0, 17.0, 19.0, 21.0] + [0.0] * 124)   # ulp 2 in [16, 32): 17 -> 16, 19 -> 20, 21 -> 20
    q3, _ = O.fp8_quant_token(ties.view(1, 128))
    assert q3.float().view(-1)[:4].tolist() == [448.0, 16.0, 20.0, 20.0]
    # scaling the row by a power of two scales the scale and leaves the codes alone
    q4, s4 = O.fp8_quant_token(x[2:3] * 8)
    assert torch.equal(q4.view(torch.uint8), q[2:3].view(torch.uint8)) and s4.item() == s[2].item() * 8
