"""Merge of the split-KV partials fused with the value up-projection, through the C-ABI, against the oracle chain
absorbed decode (fp32) -> _v_up_proj (fp32), and against the unfused path of the library (decode, then torch.bmm).

Bar: the fused kernel rounds the merged attention row to bf16 before the MFMA, exactly as the unfused path does, so
against the unfused path only the accumulation order of the 512-term sums differs (fp32): max-abs 2^-7 relative to the
largest |out| of the case.  Against the fp32 oracle the attention tolerance carries over: W_UV ~ N(0, 0.02) scales
the 2e-2 / 2e-3 bar of the attention rows by the column norm of W_UV (0.02 * sqrt(512) = 0.45)."""
import pytest
import torch

from oracle import mla_oracle as O
from tests.conftest import attn_close

pytestmark = pytest.mark.gpu


def _w_uv(n, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, 512, 128, generator=g) * 0.02).bfloat16()


@pytest.mark.parametrize("batch,heads,q_len,lo,hi,splits", [(4, 16, 1, 128, 1024, 2), (64, 128, 1, 100, 700, 4),
                                                            (5, 128, 2, 1, 600, 3), (19, 40, 1, 50, 400, None),
                                                            (2, 128, 1, 3000, 6000, 11), (3, 128, 1, 50, 300, 9),
                                                            (2, 128, 1, 3000, 6000, 40), (125, 128, 2, 2, 200, 1), (150, 128, 2, 2, 200, 1)])
def test_fused_merge_and_up_projection(dev, batch, heads, q_len, lo, hi, splits):
    """Up to 11 chunks per sequence and 256 tokens the fused kernel runs (rows of 7..12 partials take two rounds; the
    case with more chunks than work units has empty chunks); the last two cases take the other route behind the same
    call (separate merge, then the library GEMM): many partials per row, and more than 256 tokens."""
    from omni_npu_amd import kernels as K
    c = O.make_decode_case(batch, heads, lo, hi, seed=7 * batch + q_len, q_len=q_len)
    w = _w_uv(heads, seed=batch)
    t = batch * q_len
    args = [c[k].to(dev) for k in ("q_nope", "q_rope", "nope", "rope", "block_table", "seq_lens")]
    out = torch.full((t, heads * 128), float("nan"), dtype=torch.bfloat16, device=dev)
    K.decode(*args, c["scale"], out, q_len=q_len, num_splits=splits, w_uv=w.to(dev))
    # unfused path of the library
    o = torch.empty(t, heads, 512, dtype=torch.bfloat16, device=dev)
    K.decode(*args, c["scale"], o, q_len=q_len, num_splits=splits)
    unfused = torch.bmm(o.transpose(0, 1).float(), w.to(dev).float()).transpose(0, 1).reshape(t, heads * 128)
    torch.cuda.synchronize()
    got = out.float()
    assert torch.isfinite(got).all()
    scale_ref = unfused.abs().max().item()
    assert (got - unfused).abs().max().item() <= scale_ref * 2 ** -7
    # oracle chain in fp32
    ref_o = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], c["scale"])
    ref = torch.bmm(ref_o.transpose(0, 1), w.float()).transpose(0, 1).reshape(t, heads * 128)
    attn_close(out, ref, 2e-2 * 0.45, 2e-3 * 1.5)


def test_fused_up_projection_identity_weight_returns_the_attention_rows(dev):
    """W_UV[n] = first 128 columns of the identity: the output must be the bf16 attention rows' first 128 columns,
    bit for bit (one product per sum)."""
    from omni_npu_amd import kernels as K
    batch, heads = 6, 128
    c = O.make_decode_case(batch, heads, 64, 500, seed=3)
    w = torch.zeros(heads, 512, 128).bfloat16()
    for n in range(heads):
        off = (n * 37) % 384                                  # a different 128-column window for every head
        w[n, off:off + 128, :] = torch.eye(128).bfloat16()
    args = [c[k].to(dev) for k in ("q_nope", "q_rope", "nope", "rope", "block_table", "seq_lens")]
    out = torch.empty(batch, heads * 128, dtype=torch.bfloat16, device=dev)
    K.decode(*args, c["scale"], out, num_splits=3, w_uv=w.to(dev))
    o = torch.empty(batch, heads, 512, dtype=torch.bfloat16, device=dev)
    K.decode(*args, c["scale"], o, num_splits=3)
    torch.cuda.synchronize()
    want = torch.stack([o[:, n, (n * 37) % 384:(n * 37) % 384 + 128] for n in range(heads)], dim=1).reshape(batch, -1)
    assert torch.equal(out, want)


def test_fused_up_projection_strided_output_and_varlen_queries(dev):
    """Output written into a slice of a wider, padded buffer; query tokens given by query_start_loc with one request
    shorter than the uniform length (its missing token's row must stay untouched)."""
    from omni_npu_amd import kernels as K
    batch, heads, q_len = 3, 128, 2
    c = O.make_decode_case(batch, heads, 100, 500, seed=9, q_len=q_len)
    # W_UV as the reference derives it: a transposed view [N, 512, 128] of a [512, N, 128] tensor (row stride N * 128)
    g = torch.Generator().manual_seed(1)
    w = (torch.randn(512, heads, 128, generator=g) * 0.02).bfloat16().to(dev).transpose(0, 1)
    assert not w.is_contiguous()
    qsl = torch.tensor([0, 2, 3, 5], dtype=torch.int32)        # request 1 has one token only
    keep = torch.tensor([0, 1, 2, 4, 5])
    qn, qr = c["q_nope"][keep].contiguous(), c["q_rope"][keep].contiguous()
    t = 5
    buf = torch.full((t + 3, heads * 128 + 64), 7.0, dtype=torch.bfloat16, device=dev)
    out = buf[:t, 64:]
    K.decode(qn.to(dev), qr.to(dev), c["nope"].to(dev), c["rope"].to(dev), c["block_table"].to(dev), c["seq_lens"].to(dev),
             c["scale"], out.view(t, heads, 128), q_len=q_len, query_start_loc=qsl.to(dev), num_splits=2, w_uv=w)
    o = torch.empty(t, heads, 512, dtype=torch.bfloat16, device=dev)
    K.decode(qn.to(dev), qr.to(dev), c["nope"].to(dev), c["rope"].to(dev), c["block_table"].to(dev), c["seq_lens"].to(dev),
             c["scale"], o, q_len=q_len, query_start_loc=qsl.to(dev), num_splits=2)
    unfused = torch.bmm(o.transpose(0, 1).float(), w.float()).transpose(0, 1).reshape(t, heads * 128)
    torch.cuda.synchronize()
    assert (out.float() - unfused).abs().max().item() <= unfused.abs().max().item() * 2 ** -7
    assert (buf[t:] == 7.0).all() and (buf[:, :64] == 7.0).all()


def test_fused_up_projection_after_fp8_and_sparse_decode(dev):
    """The same fused merge after the other two split kernels: the fp8-cache decode and the row-list (sparse) decode,
    each against its own unfused path."""
    from omni_npu_amd import kernels as K
    batch, heads = 5, 128
    c = O.make_decode_case(batch, heads, 200, 900, seed=31, q_len=2)
    w = _w_uv(heads, seed=2).to(dev)
    t = batch * 2
    cache = torch.zeros(c["nope"].shape[0], 128, 656, dtype=torch.uint8, device=dev)
    K.cache_write_fp8(c["nope"].view(-1, 512).to(dev), c["rope"].view(-1, 64).to(dev),
                      torch.arange(cache.shape[0] * 128, dtype=torch.int64, device=dev), cache)
    a8 = (c["q_nope"].to(dev), c["q_rope"].to(dev), cache, c["block_table"].to(dev), c["seq_lens"].to(dev), c["scale"])
    out = torch.full((t, heads * 128), float("nan"), dtype=torch.bfloat16, device=dev)
    K.decode_fp8(*a8, out, q_len=2, num_splits=3, w_uv=w)
    o = torch.empty(t, heads, 512, dtype=torch.bfloat16, device=dev)
    K.decode_fp8(*a8, o, q_len=2, num_splits=3)
    unfused = torch.bmm(o.transpose(0, 1).float(), w.float()).transpose(0, 1).reshape(t, heads * 128)
    torch.cuda.synchronize()
    assert (out.float() - unfused).abs().max().item() <= unfused.abs().max().item() * 2 ** -7

    c1 = O.make_decode_case(4, heads, 300, 700, seed=32)
    k = 256
    rows = torch.zeros(4, k, dtype=torch.int32)
    counts = torch.zeros(4, dtype=torch.int32)
    for b in range(4):
        pos = torch.arange(0, int(c1["seq_lens"][b]), 2)[:k]
        rows[b, :pos.numel()] = O.slots_for(c1["block_table"], b, 0, int(c1["seq_lens"][b]))[pos].to(torch.int32)
        counts[b] = pos.numel()
    a_s = (c1["q_nope"].to(dev), c1["q_rope"].to(dev), c1["nope"].to(dev), c1["rope"].to(dev), rows.to(dev), counts.to(dev),
           c1["scale"])
    out_s = torch.full((4, heads * 128), float("nan"), dtype=torch.bfloat16, device=dev)
    K.sparse_decode(*a_s, out_s, num_splits=4, w_uv=w)
    o_s = torch.empty(4, heads, 512, dtype=torch.bfloat16, device=dev)
    K.sparse_decode(*a_s, o_s, num_splits=4)
    unfused_s = torch.bmm(o_s.transpose(0, 1).float(), w.float()).transpose(0, 1).reshape(4, heads * 128)
    torch.cuda.synchronize()
    assert (out_s.float() - unfused_s).abs().max().item() <= unfused_s.abs().max().item() * 2 ** -7
