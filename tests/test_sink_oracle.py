"""Pins for the static-sink / sliding-window functions of the oracle.  The reference (attention/backends/mla.py:463-560,
:705-779) computes two attentions with LSE and merges them; these checks use formulas that share nothing with that
construction: one softmax over the union of the keys (per-token loop, float64), torch's scaled_dot_product_attention
with an explicit boolean mask, and the special cases in which the variant must reduce to the plain decode."""
import math

import pytest
import torch

from oracle import mla_oracle as O


def _sink_case(batch, heads, lo, hi, sink_len, q_len, seed):
    """A decode case whose block tables carry sink_len / 128 shared sink pages in front of every row."""
    c = O.make_decode_case(batch, heads, lo, hi, seed=seed, q_len=q_len, extra_blocks=sink_len // O.PAGE)
    nsb = sink_len // O.PAGE
    nblk = c["nope"].shape[0]
    sink_pages = torch.arange(nblk - nsb, nblk, dtype=torch.int32)        # the extra pages, never in a sequence's table
    bt = torch.cat([sink_pages.view(1, -1).expand(batch, -1), c["block_table"]], 1).contiguous()
    return c, bt


def _union_brute_force(c, bt, sink_len, window, q_len):
    """softmax over {sink keys} U {visible keys of the sequence}, float64, one (token, head) row at a time."""
    kc = c["nope"].reshape(-1, 512).double()
    kr = c["rope"].reshape(-1, 64).double()
    t, n, _ = c["q_nope"].shape
    out = torch.zeros(t, n, 512, dtype=torch.float64)
    for b in range(len(c["seq_lens"])):
        L = int(c["seq_lens"][b])
        for i in range(q_len):
            last = L - q_len + i                                            # newest key this token sees
            first = 0 if window is None else max(0, last - window + 1)
            pos = list(range(sink_len)) + [sink_len + j for j in range(first, last + 1)]
            rows = torch.tensor([int(bt[b, p // 128]) * 128 + p % 128 for p in pos])
            for h in range(n):
                tk = b * q_len + i
                sc = (kc[rows] @ c["q_nope"][tk, h].double() + kr[rows] @ c["q_rope"][tk, h].double()) * c["scale"]
                out[tk, h] = torch.softmax(sc, 0) @ kc[rows]
    return out


@pytest.mark.parametrize("sink_len,window,q_len", [(128, None, 1), (128, 40, 1), (256, 7, 2), (128, 1, 3), (128, 1000, 2)])
def test_sink_decode_is_one_softmax_over_the_union(sink_len, window, q_len):
    c, bt = _sink_case(3, 4, 20, 300, sink_len, q_len, seed=sink_len + q_len)
    got = O.sink_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], bt, c["seq_lens"], sink_len, c["scale"], window)
    want = _union_brute_force(c, bt, sink_len, window, q_len)
    assert (got.double() - want).abs().max() < 2e-5


def test_sink_decode_without_window_is_plain_decode_over_the_longer_table():
    c, bt = _sink_case(4, 8, 50, 400, 256, 2, seed=3)
    got = O.sink_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], bt, c["seq_lens"], 256, c["scale"])
    plain = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], bt, c["seq_lens"] + 256, c["scale"])
    assert (got - plain).abs().max() < 2e-5


def test_window_not_shorter_than_the_sequence_changes_nothing():
    c, bt = _sink_case(3, 4, 30, 200, 128, 2, seed=5)
    a = O.sink_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], bt, c["seq_lens"], 128, c["scale"], window=None)
    b = O.sink_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], bt, c["seq_lens"], 128, c["scale"], window=200)
    assert torch.equal(a, b)
    d = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], c["scale"])
    e = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], c["scale"],
                          window=10 ** 6)
    assert torch.equal(d, e)


def test_sink_len_must_be_whole_pages():
    c, bt = _sink_case(1, 2, 10, 20, 128, 1, seed=0)
    with pytest.raises(ValueError, match="must align with block size"):
        O.sink_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], bt, c["seq_lens"], 100, c["scale"])


def test_windowed_varlen_attention_matches_sdpa_with_a_band_mask():
    g = torch.Generator().manual_seed(2)
    n, sq, sk, w = 3, 37, 50, 9
    qn, qp = torch.randn(sq, n, 128, generator=g), torch.randn(sq, n, 64, generator=g)
    kn, kp, v = torch.randn(sk, n, 128, generator=g), torch.randn(sk, 64, generator=g), torch.randn(sk, n, 128, generator=g)
    scale = 1 / math.sqrt(192)
    out, lse = O.attention_varlen(qn, qp, kn, kp, v, [0, sq], [0, sk], scale, True, window=w)
    i, j = torch.arange(sq).view(-1, 1), torch.arange(sk).view(1, -1)
    mask = (j <= i + sk - sq) & (j >= i + sk - sq - (w - 1))              # pre_tokens = w - 1, next_tokens = 0
    q = torch.cat([qn, qp], -1).transpose(0, 1)
    k = torch.cat([kn, kp.unsqueeze(1).expand(-1, n, -1)], -1).transpose(0, 1)
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v.transpose(0, 1), attn_mask=mask, scale=scale)
    assert (out - want.transpose(0, 1)).abs().max() < 2e-5
    assert int(mask.sum(1).max()) == w and int(mask.sum(1).min()) == w     # every row of this case has a full window


@pytest.mark.parametrize("window", [None, 6, 64])
def test_sink_prefill_is_sdpa_over_sink_plus_band(window):
    g = torch.Generator().manual_seed(4)
    n, s_len = 2, 8
    cu_q = [0, 5, 30, 31]
    t = cu_q[-1]
    q = torch.randn(t, n, 192, generator=g)
    kv_c, k_pe = torch.randn(t, 512, generator=g), torch.randn(t, 64, generator=g)
    sink_c, sink_pe = torch.randn(s_len, 512, generator=g), torch.randn(s_len, 64, generator=g)
    w_kv_b = torch.randn(512, n * 256, generator=g) / math.sqrt(512)
    scale = 1 / math.sqrt(192)
    got = O.sink_prefill(q, kv_c, k_pe, w_kv_b, sink_c, sink_pe, cu_q, scale, window).view(t, n, 128)
    for b in range(3):
        q0, q1 = cu_q[b], cu_q[b + 1]
        s = q1 - q0
        lat = torch.cat([sink_c, kv_c[q0:q1]])
        pe = torch.cat([sink_pe, k_pe[q0:q1]])
        kn, v = O.kv_up_proj(lat, w_kv_b, n, 128, 128)
        k = torch.cat([kn, pe.unsqueeze(1).expand(-1, n, -1)], -1).transpose(0, 1)
        i, j = torch.arange(s).view(-1, 1), torch.arange(s_len + s).view(1, -1)
        mask = j <= i + s_len
        if window is not None:
            mask &= (j < s_len) | (j - s_len > i - window)
        want = torch.nn.functional.scaled_dot_product_attention(q[q0:q1].transpose(0, 1), k, v.transpose(0, 1),
                                                                attn_mask=mask, scale=scale)
        assert (got[q0:q1] - want.transpose(0, 1)).abs().max() < 3e-5
