"""Pins of the oracle's RMSNorm / rotary embedding / fused cache write (no GPU): library routine, float64 loops and the
invariants a rotation must satisfy, chosen so that a wrong sign, a swapped pair or a wrong table entry fails."""
import math

import torch

from oracle import mla_oracle as O


def _case(t=7, seed=0):
    g = torch.Generator().manual_seed(seed)
    kv = torch.randn(t, 576, generator=g).bfloat16()
    gamma = (1 + 0.1 * torch.randn(512, generator=g)).bfloat16()
    pos = torch.randint(0, 5000, (t,), generator=g)
    return kv, gamma, pos


def test_rms_norm_matches_library_and_loop():
    kv, gamma, _ = _case()
    x = kv[:, :512]
    got = O.rms_norm(x, gamma, 1e-6)
    lib = torch.nn.functional.rms_norm(x.double(), (512,), gamma.double(), 1e-6).bfloat16()
    assert torch.equal(got, lib)
    row = x[3].double()
    want = row / math.sqrt(float((row * row).sum()) / 512 + 1e-6) * gamma.double()
    assert torch.equal(got[3], want.bfloat16())
    # eps matters for a tiny row, and an all-zero row stays zero
    z = torch.zeros(1, 512).bfloat16()
    assert (O.rms_norm(z, gamma, 1e-6) == 0).all()
    tiny = torch.full((1, 512), 1e-4).bfloat16()
    assert not torch.equal(O.rms_norm(tiny, gamma, 1e-6), O.rms_norm(tiny, gamma, 1e-12))


def test_rope_float64_loop_both_layouts():
    kv, _, pos = _case()
    x = kv[:, 512:]
    for layout in ("half", "repeat"):
        cos, sin = O.rope_tables(pos, layout=layout)
        half = O.interleave_rope(x, cos, sin, table=layout)
        inter = O.interleave_rope(x, cos, sin, table=layout, interleaved_out=True)
        for t in (0, 5):
            for i in (0, 13, 31):
                e = i if layout == "half" else 2 * i
                c, s = float(cos[t, e]), float(sin[t, e])
                a, b = float(x[t, 2 * i]), float(x[t, 2 * i + 1])
                o1 = torch.tensor(a * c - b * s, dtype=torch.float64).bfloat16()
                o2 = torch.tensor(b * c + a * s, dtype=torch.float64).bfloat16()
                assert half[t, i] == o1 and half[t, 32 + i] == o2
                assert inter[t, 2 * i] == o1 and inter[t, 2 * i + 1] == o2
    # the two table layouts carry the same numbers: results agree
    ch, sh = O.rope_tables(pos, layout="half")
    cr, sr = O.rope_tables(pos, layout="repeat")
    assert torch.equal(O.interleave_rope(x, ch, sh, "half"), O.interleave_rope(x, cr, sr, "repeat"))


def test_rope_is_a_rotation():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 3, 64, generator=g).bfloat16()
    # position 0: cos = 1, sin = 0 -> de-interleave only
    c0, s0 = O.rope_tables(torch.zeros(5, dtype=torch.long))
    out0 = O.interleave_rope(x, c0, s0)
    assert torch.equal(out0, torch.cat((x[..., 0::2], x[..., 1::2]), -1))
    # pair norms are preserved (fp32 tables so that only the final rounding remains)
    pos = torch.tensor([1, 17, 300, 4095, 9999])
    c, s = O.rope_tables(pos, dtype=torch.float32)
    out = O.interleave_rope(x.double(), c, s)
    n_in = x[..., 0::2].double() ** 2 + x[..., 1::2].double() ** 2
    n_out = out[..., :32] ** 2 + out[..., 32:] ** 2
    assert torch.allclose(n_in, n_out, rtol=1e-6, atol=1e-9)
    # q . k after rotation depends on the position difference only
    q, k = torch.randn(1, 64, generator=g).double(), torch.randn(1, 64, generator=g).double()
    def dot(pq, pk):
        cq, sq = O.rope_tables(torch.tensor([pq]), dtype=torch.float64)
        ck, sk = O.rope_tables(torch.tensor([pk]), dtype=torch.float64)
        return float((O.interleave_rope(q, cq, sq) * O.interleave_rope(k, ck, sk)).sum())
    assert abs(dot(100, 40) - dot(1060, 1000)) < 1e-3
    assert abs(dot(100, 40) - dot(100, 41)) > 1e-3


def test_fused_oracle_is_the_composition_and_skips_pad_slots():
    kv, gamma, pos = _case(t=6, seed=2)
    cos, sin = O.rope_tables(pos)
    nope = torch.zeros(2, 128, 512).bfloat16()
    rope = torch.zeros(2, 128, 64).bfloat16()
    slots = torch.tensor([5, 130, -1, 255, 0, -1])
    k_pe, kv_a = O.kv_rmsnorm_rope_cache(kv, gamma, cos, sin, slots, nope, rope, 1e-6)
    assert torch.equal(kv_a, O.rms_norm(kv[:, :512], gamma, 1e-6))
    assert torch.equal(k_pe, O.interleave_rope(kv[:, 512:], cos, sin))
    flat_n, flat_r = nope.view(-1, 512), rope.view(-1, 64)
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            assert torch.equal(flat_n[s], kv_a[t]) and torch.equal(flat_r[s], k_pe[t])
    untouched = torch.ones(256, dtype=torch.bool)
    untouched[[5, 130, 255, 0]] = False
    assert (flat_n[untouched] == 0).all() and (flat_r[untouched] == 0).all()


def test_rotary_mul_float64_loop_library_rotate_half_and_the_interleaved_form():
    """The half-rotation pairing (torch_npu.npu_rotary_mul in the indexer, npu_dsa.py:120, 130): entry by entry in
    float64, against the transformers library's rotate_half formulation, and as the interleaved form on permuted input."""
    g = torch.Generator().manual_seed(21)
    x = torch.randn(6, 3, 64, generator=g).bfloat16()
    pos = torch.tensor([0, 1, 17, 300, 4095, 9999])
    cos, sin = O.rope_tables(pos)
    out = O.rotary_mul(x, cos, sin)
    for t in (0, 2, 5):
        for i in (0, 13, 31):
            c, s = float(cos[t, i]), float(sin[t, i])
            a, b = float(x[t, 1, i]), float(x[t, 1, 32 + i])
            assert out[t, 1, i] == torch.tensor(a * c - b * s, dtype=torch.float64).bfloat16()
            assert out[t, 1, 32 + i] == torch.tensor(b * c + a * s, dtype=torch.float64).bfloat16()
    # library routine: q * cos + rotate_half(q) * sin with full-width rows cat(c, c)
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    xd = x.double().transpose(0, 1).unsqueeze(0)                        # [1, heads, tokens, 64]
    lib, _ = apply_rotary_pos_emb(xd, xd, cos.double().unsqueeze(0), sin.double().unsqueeze(0))
    assert torch.equal(lib.squeeze(0).transpose(0, 1).bfloat16(), out)
    # the same rotation as the interleaved pairing applied to the interleaved arrangement of the same numbers
    inter = torch.stack((x[..., :32], x[..., 32:]), -1).reshape(x.shape)
    assert torch.equal(O.interleave_rope(inter, cos, sin), out)
    # the 'repeat' table layout carries the same numbers
    cr, sr = O.rope_tables(pos, layout="repeat")
    assert torch.equal(O.rotary_mul(x, cr, sr, "repeat"), out)
