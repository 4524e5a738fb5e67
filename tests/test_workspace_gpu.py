"""Scratch memory under HIP graphs and under long prefills: a captured graph keeps writing into the buffer it captured
after a later, larger call made the wrapper allocate a new one; a sparse prefill of a few thousand tokens runs in bounded
scratch and matches the oracle on sampled tokens; row counts beyond the row list are clamped."""
import pytest
import torch

from oracle import mla_oracle as O

pytestmark = pytest.mark.gpu


def _case(dev, batch, lo, hi, seed, heads=128):
    c = O.make_decode_case(batch, heads, lo, hi, seed=seed)
    g = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in c.items()}
    return c, g


def test_graph_captured_with_a_small_workspace_survives_a_larger_later_call(dev):
    from omni_npu_amd import kernels as K
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        ca, ga = _case(dev, 3, 100, 700, seed=1)
        out_a = torch.zeros(3, 128, 512, dtype=torch.bfloat16, device=dev)

        def step_a():
            K.decode(ga["q_nope"], ga["q_rope"], ga["nope"], ga["rope"], ga["block_table"], ga["seq_lens"], ca["scale"], out_a,
                     num_splits=4)

        step_a()                                              # warm-up: allocates the (small) scratch of this stream
        torch.cuda.synchronize()
        key = (dev.index, side.cuda_stream, "decode")
        small = K._workspaces[key][-1]
        small_ptr, n_before = small.data_ptr(), len(K._workspaces[key])
        eager_a = out_a.clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step_a()
        # descriptor B needs much more scratch: the wrapper must allocate next to the old buffer, not replace it
        cb, gb = _case(dev, 48, 200, 900, seed=2)
        out_b = torch.zeros(48, 128, 512, dtype=torch.bfloat16, device=dev)
        K.decode(gb["q_nope"], gb["q_rope"], gb["nope"], gb["rope"], gb["block_table"], gb["seq_lens"], cb["scale"], out_b,
                 num_splits=4)
        torch.cuda.synchronize()
        bufs = K._workspaces[key]
        assert len(bufs) == n_before + 1 and bufs[-1].numel() > small.numel()
        assert bufs[n_before - 1] is small and small.data_ptr() == small_ptr      # still alive, at its address
        # memory churn: whatever the allocator hands out now must not be the old scratch
        junk = [torch.full((small.numel(),), 0x7f, dtype=torch.uint8, device=dev) for _ in range(4)]
        for rep in range(3):
            out_a.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out_a, eager_a), f"replay {rep} of the older graph differs from the eager step"
            K.decode(gb["q_nope"], gb["q_rope"], gb["nope"], gb["rope"], gb["block_table"], gb["seq_lens"], cb["scale"], out_b,
                     num_splits=4)                            # eager work between the replays
            torch.cuda.synchronize()
        assert all(int(j[0]) == 0x7f and int(j[-1]) == 0x7f for j in junk)
        ref_b = O.absorbed_decode(cb["q_nope"], cb["q_rope"], cb["nope"], cb["rope"], cb["block_table"], cb["seq_lens"], cb["scale"])
        assert (out_b.float().cpu() - ref_b).abs().max() <= 2e-2
    torch.cuda.current_stream().wait_stream(side)


def test_sparse_prefill_of_a_few_thousand_tokens_in_bounded_scratch(dev):
    """3000 one-token rows x 128 heads: more than one launch under SPARSE_WORKSPACE_CAP; sampled tokens against the oracle,
    the fused up-projection against the unfused result."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(5)
    t, n, k, pages = 3000, 128, 96, 24
    nope = torch.randn(pages, 128, 512, generator=g).bfloat16()
    rope = torch.randn(pages, 128, 64, generator=g).bfloat16()
    q_nope = torch.randn(t, n, 512, generator=g).bfloat16()
    q_rope = torch.randn(t, n, 64, generator=g).bfloat16()
    total = pages * 128
    pos = torch.stack([torch.randperm(total, generator=g)[:k] for _ in range(t)]).to(torch.int32)
    counts = torch.randint(1, k + 1, (t,), generator=g, dtype=torch.int32)
    counts[7] = k + 50                                        # beyond the row list: clamped to k
    scale = 1.0 / 192 ** 0.5
    need_all = K._lib.load().mla_decode_workspace_bytes(t, 1, n, 1)
    assert need_all > K.SPARSE_WORKSPACE_CAP                   # one launch would not fit under the cap
    out = torch.full((t, n, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    lse = torch.full((t, n), float("nan"), dtype=torch.float32, device=dev)
    K.sparse_decode(q_nope.to(dev), q_rope.to(dev), nope.to(dev), rope.to(dev), pos.to(dev), counts.to(dev), scale, out,
                    lse_out=lse, num_splits=1)
    torch.cuda.synchronize()
    key = (dev.index, torch.cuda.current_stream().cuda_stream, "decode")
    assert K._workspaces[key][-1].numel() <= max(K.SPARSE_WORKSPACE_CAP, K._workspaces[key][0].numel()) * 3 // 2
    assert torch.isfinite(out.float()).all()
    sample = [0, 1, 7, 1007, 1008, 1500, 2015, 2016, 2999]     # both sides of the launch borders (1008 tokens per launch)
    bt = torch.arange(pages, dtype=torch.int32).repeat(len(sample), 1)
    idx = torch.full((len(sample), k), -1, dtype=torch.int32)
    for j, tok in enumerate(sample):
        c = min(int(counts[tok]), k)
        idx[j, :c] = pos[tok, :c]
    ref, ref_lse = O.sparse_decode(q_nope[sample], q_rope[sample], nope, rope, bt, torch.full((len(sample),), total), idx, scale,
                                   return_lse=True)
    got = out[sample].float().cpu()
    assert (got - ref).abs().max() <= 2e-2 and ((got - ref).abs().mean() / ref.abs().mean()) <= 2e-3
    assert torch.allclose(lse[sample].cpu(), ref_lse, atol=2e-2, rtol=0)
    # the fused up-projection over the same tiled launches
    w = (torch.randn(n, 512, 128, generator=g) * 0.02).bfloat16()
    out_v = torch.full((t, n * 128), float("nan"), dtype=torch.bfloat16, device=dev)
    K.sparse_decode(q_nope.to(dev), q_rope.to(dev), nope.to(dev), rope.to(dev), pos.to(dev), counts.to(dev), scale, out_v,
                    num_splits=1, w_uv=w.to(dev))
    ref_v = torch.bmm(ref.transpose(0, 1), w.float()).transpose(0, 1).reshape(len(sample), n * 128)
    got_v = out_v[sample].float().cpu()
    assert (got_v - ref_v).abs().max() <= 2e-2 * 0.45 and ((got_v - ref_v).abs().mean() / ref_v.abs().mean()) <= 3e-3
