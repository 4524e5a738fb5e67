"""Host-side contract of the plugin boundary, without a GPU and without vLLM: what the reference pins with its
mock-based unit tests (tests/unit/platform/test_platform.py, test_vllm_plugin.py, tests/unit/attention/backends/
test_mla.py:151-188, test_dsa.py:11-46, 68-164, 208-247, tests/unit/compilation/test_acl_graph.py:176-197),
re-stated for this package's classes."""
from types import SimpleNamespace

import pytest
import torch

from omni_npu_amd import _vllm_compat as V
from omni_npu_amd import platform as P
from omni_npu_amd import vllm_plugin
from omni_npu_amd.attention.backends import dsa, mla
from omni_npu_amd.compilation.acl_graph import ACLGraphWrapper, HIPGraphWrapper
from omni_npu_amd.worker import hip_worker


def _cfg(max_num_seqs=8, cap=None, spec=None, kv_transfer=None):
    return SimpleNamespace(
        scheduler_config=SimpleNamespace(max_num_seqs=max_num_seqs),
        model_config=SimpleNamespace(max_model_len=4096, dtype=torch.bfloat16),
        cache_config=SimpleNamespace(block_size=128, cache_dtype="auto"),
        parallel_config=SimpleNamespace(cp_kv_cache_interleave_size=1, decode_context_parallel_size=1, worker_cls=None),
        compilation_config=SimpleNamespace(max_cudagraph_capture_size=cap, pass_config=SimpleNamespace(
            fuse_norm_quant=True, fuse_act_quant=True, fuse_attn_quant=True)),
        kv_transfer_config=kv_transfer, speculative_config=spec)


def _common(q_lens, seq_lens, page=128):
    qsl = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    sl = torch.tensor(seq_lens, dtype=torch.int32)
    nblk = [(s + page - 1) // page for s in seq_lens]
    bt = torch.zeros(len(q_lens), max(nblk), dtype=torch.int32)
    o = 0
    for i, n in enumerate(nblk):
        bt[i, :n] = torch.arange(o, o + n)
        o += n
    t = int(qsl[-1])
    return V.CommonAttentionMetadata(query_start_loc=qsl, query_start_loc_cpu=qsl.clone(), seq_lens=sl, seq_lens_cpu=sl.clone(),
                                     num_computed_tokens_cpu=sl - torch.tensor(q_lens, dtype=torch.int32), num_reqs=len(q_lens),
                                     num_actual_tokens=t, max_query_len=max(q_lens), max_seq_len=max(seq_lens),
                                     block_table_tensor=bt, slot_mapping=torch.arange(t, dtype=torch.int64))


# ---- plugin + platform ---------------------------------------------------------------------------------
def test_plugin_returns_none_without_a_gfx950_device():
    assert vllm_plugin.plugin() is None                      # this box has no GPU


def test_plugin_returns_platform_path_on_gfx950(monkeypatch):
    monkeypatch.setattr(torch.version, "hip", "7.0", raising=False)
    monkeypatch.setattr(torch.cuda, "device_count", lambda: 1)
    monkeypatch.setattr(torch.cuda, "get_device_properties", lambda i: SimpleNamespace(gcnArchName="gfx950:sramecc+:xnack-"))
    assert vllm_plugin.plugin() == "omni_npu_amd.platform.MI355XPlatform"
    monkeypatch.setattr(torch.cuda, "get_device_properties", lambda i: SimpleNamespace(gcnArchName="gfx942"))
    assert vllm_plugin.plugin() is None


def test_platform_selection_and_config_defaults():
    plat = P.MI355XPlatform
    assert P.NPUPlatform is plat
    sel = lambda **kw: plat.get_attn_backend_cls(None, 576, torch.bfloat16, None, 128, has_sink=False, **kw)
    assert sel(use_mla=True, use_sparse=True) == "omni_npu_amd.attention.backends.dsa.NPUDSABackend"
    assert sel(use_mla=True, use_sparse=False) == "omni_npu_amd.attention.backends.mla.NPUMLABackend"
    with pytest.raises(NotImplementedError):
        sel(use_mla=False, use_sparse=False)
    assert plat.support_static_graph_mode() is True
    assert plat.get_static_graph_wrapper_cls() == "omni_npu_amd.compilation.acl_graph.HIPGraphWrapper"
    assert plat.dist_backend == "nccl" and plat.device_type == "cuda"
    cfg = _cfg()
    cfg.cache_config.block_size = None
    plat.check_and_update_config(cfg)
    assert cfg.parallel_config.worker_cls == "omni_npu_amd.worker.hip_worker.HIPWorker"
    assert cfg.cache_config.block_size == 128
    pc = cfg.compilation_config.pass_config
    assert not (pc.fuse_norm_quant or pc.fuse_act_quant or pc.fuse_attn_quant)
    cfg.cache_config.block_size = 64
    plat.check_and_update_config(cfg)
    assert cfg.cache_config.block_size == 64                 # an explicit value is left alone
    # every dotted path the platform hands to vLLM resolves to a class of this package
    import importlib
    for path in (sel(use_mla=True, use_sparse=True), sel(use_mla=True, use_sparse=False),
                 plat.get_static_graph_wrapper_cls(), cfg.parallel_config.worker_cls):
        mod, name = path.rsplit(".", 1)
        assert hasattr(importlib.import_module(mod), name)


# ---- backends: names and cache reshape ---------------------------------------------------------------------
def test_mla_backend_contract_and_reshape():
    B = mla.NPUMLABackend
    assert B.get_name() == "NPUMLA" and B.get_impl_cls() is mla.NPUMLAImpl
    assert B.get_builder_cls() is mla.NPUMLAMetadataBuilder and B.get_metadata_cls() is mla.NPUMLAMetadata
    nb, bs = 4, 128
    raw = torch.zeros(nb * bs * 576 * 2, dtype=torch.uint8)
    nope, rope = B.reshape_kv_cache(raw, nb, bs, 1, 576, dtype=torch.bfloat16)
    assert nope.shape == (nb, bs, 512) and rope.shape == (nb, bs, 64)
    assert nope.dtype == rope.dtype == torch.bfloat16 and nope.is_contiguous() and rope.is_contiguous()
    # all nope pages first, then all rope pages, in the one allocation
    assert nope.data_ptr() == raw.data_ptr() and rope.data_ptr() == raw.data_ptr() + nb * bs * 512 * 2
    with pytest.raises(RuntimeError, match="expected sizes for KV cache"):
        B.reshape_kv_cache(raw[:-2], nb, bs, 1, 576, dtype=torch.bfloat16)
    (c8,) = B.reshape_kv_cache(torch.zeros(nb * bs * 656, dtype=torch.uint8), nb, bs, 1, 656, dtype=torch.uint8)
    assert c8.shape == (nb, bs, 656) and c8.dtype == torch.uint8
    with pytest.raises(RuntimeError):
        B.reshape_kv_cache(torch.zeros(nb * bs * 656 - 1, dtype=torch.uint8), nb, bs, 1, 656, dtype=torch.uint8)


def test_dsa_backend_contract_and_reshape():
    B = dsa.NPUDSABackend
    assert B.get_name() == "NPUDSA" and B.get_impl_cls() is dsa.NPUDSAImpl
    nb, bs = 3, 128
    raw = torch.zeros(nb * bs * 704 * 2, dtype=torch.uint8)
    a, b, c = B.reshape_kv_cache(raw, nb, bs, 1, 704, dtype=torch.bfloat16)
    assert a.shape == (nb, bs, 1, 512) and b.shape == (nb, bs, 1, 64) and c.shape == (nb, bs, 1, 128)
    with pytest.raises(RuntimeError, match="expected sizes for KV cache"):
        B.reshape_kv_cache(raw[:-2], nb, bs, 1, 704, dtype=torch.bfloat16)
    k8, ks = dsa.indexer_cache_views(c)
    assert k8.shape == (nb, bs, 128) and k8.dtype == torch.uint8 and ks.shape == (nb, bs) and ks.dtype == torch.float32
    assert k8.data_ptr() == c.data_ptr() and ks.data_ptr() == c.data_ptr() + bs * 128
    assert k8.stride(0) == bs * 256 and ks.stride(0) == bs * 64          # one 32 KiB page region per block


def test_kv_spec_sizes():
    assert hip_worker.kv_cache_dtype_and_head_size("auto", torch.bfloat16, 576) == (torch.bfloat16, 576)
    assert hip_worker.kv_cache_dtype_and_head_size("fp8", torch.bfloat16, 576) == (torch.uint8, 656)
    spec = V.MLAAttentionSpec(block_size=128, num_kv_heads=1, head_size=576 + 128, dtype=torch.bfloat16)
    assert spec.page_size_bytes == 128 * 704 * 2


# ---- builders ---------------------------------------------------------------------------------------------------
def test_mla_builder_decode_metadata_stays_on_device_tensors():
    spec = V.AttentionSpec(128, 1, 576, torch.bfloat16)
    b = mla.NPUMLAMetadataBuilder(spec, ["l0"], _cfg(cap=4), torch.device("cpu"))
    assert b.reorder_batch_threshold == 4                    # raised to the largest capture size (mla.py:119-120)
    assert b._cudagraph_support == V.AttentionCGSupport.ALWAYS and b.supports_uniform_spec_as_decode
    m = b.build(0, _common([2, 2, 2], [300, 130, 2]))
    assert (m.num_decodes, m.num_prefills, m.num_decode_tokens) == (3, 0, 6)
    d = m.decode
    assert d.q_len == 2 and d.query_start_loc is None and d.seq_lens.dtype == torch.int32
    assert d.seq_lens_list == [300, 130, 2] and d.query_cumlens_list == [2, 4, 6]
    m = b.build(0, _common([1, 3, 2], [50, 60, 70]))         # ragged decode batch keeps the start offsets
    assert m.decode.q_len == 3 and m.decode.query_start_loc.tolist() == [0, 1, 4, 6]


def test_mla_builder_prefill_and_chunked_context_schedule():
    spec = V.AttentionSpec(128, 1, 576, torch.bfloat16)
    b = mla.NPUMLAMetadataBuilder(spec, ["l0"], _cfg(), torch.device("cpu"))
    b.chunked_prefill_workspace_size = 64                   # 2 requests with context -> 32 tokens per chunk
    m = b.build(0, _common([1, 16, 16], [40, 64, 64]))
    assert (m.num_decodes, m.num_prefills, m.num_decode_tokens) == (1, 2, 1)
    p = m.prefill
    assert p.query_start_loc.tolist() == [0, 16, 32] and p.query_start_loc_list == [0, 16, 32]
    assert p.query_cumlens == [1, 17, 33] and p.max_query_len == 16
    cc = p.chunked_context                                   # context 48 = chunks [32, 16] (test_mla_chunked_prefill.py:267-272)
    assert cc.seq_tot == [64, 32] and cc.cu_seq_lens.tolist() == [[0, 32, 64], [0, 16, 32]]
    assert cc.starts.tolist() == [[0, 0], [32, 32]] and cc.workspace.shape[1] == 576
    cfg = _cfg()                                            # a forbidden builder configuration (mla.py:110-117)
    cfg.parallel_config.cp_kv_cache_interleave_size = 2
    with pytest.raises(ValueError, match="cp_kv_cache_interleave_size"):
        mla.NPUMLAMetadataBuilder(spec, ["l0"], cfg, torch.device("cpu"))


def test_dsa_builder_behaviour():
    spec = V.AttentionSpec(128, 1, 704, torch.bfloat16)
    b = dsa.NPUDSAMetadataBuilder(spec, ["l0"], _cfg(spec=SimpleNamespace(num_speculative_tokens=1),
                                                      kv_transfer=object()), torch.device("cpu"))
    assert b.uniform_decode_query_len == 2 and b._cudagraph_support == V.AttentionCGSupport.UNIFORM_BATCH
    m = b.build(0, _common([2, 2], [100, 200]))
    assert m.decode.seq_lens.tolist() == [100, 200] and m.decode.query_cumlens.tolist() == [2, 4] and m.decode.q_len == 2
    c = _common([2, 2, 2], [100, 200, 300])
    c.slot_mapping = c.slot_mapping[:5]                      # short by one: padded with PAD_SLOT_ID (dsa.py:172-177)
    m = b.build(0, c)
    assert m.slot_mapping.tolist()[-1] == -1 and m.slot_mapping.numel() == 6
    b2 = dsa.NPUDSAMetadataBuilder(spec, ["l0"], _cfg(), torch.device("cpu"))
    m = b2.build(0, _common([7, 5], [7, 5]))                 # pure prefill
    assert m.prefill.seq_lens.tolist() == [7, 5] and m.prefill.query_cumlens.tolist() == [7, 12]
    with pytest.raises(RuntimeError, match="Chunked prefill is not enabled"):
        b2.build(0, _common([4, 4], [40, 4]))                # a prefill with cached context
    cfg = _cfg()
    cfg.parallel_config.decode_context_parallel_size = 2
    with pytest.raises(ValueError, match="DCP"):
        dsa.NPUDSAMetadataBuilder(spec, ["l0"], cfg, torch.device("cpu"))


# ---- impls: validation, profile run -------------------------------------------------------------------------------
def _impl(cls, **over):
    kw = dict(num_heads=8, head_size=576, scale=0.1, num_kv_heads=1, alibi_slopes=None, sliding_window=None,
              kv_cache_dtype="auto", logits_soft_cap=None, attn_type=V.AttentionType.DECODER,
              kv_sharing_target_layer_name=None, q_lora_rank=None, kv_lora_rank=512, qk_nope_head_dim=128,
              qk_rope_head_dim=64, qk_head_dim=192, v_head_dim=128, kv_b_proj=None)
    kw.update(over)
    return cls(**kw)


@pytest.mark.parametrize("cls", [mla.NPUMLAImpl, dsa.NPUDSAImpl])
def test_impl_rejects_unsupported_features(cls):
    _impl(cls)
    with pytest.raises(NotImplementedError):
        _impl(cls, alibi_slopes=[0.1])
    with pytest.raises(NotImplementedError):
        _impl(cls, logits_soft_cap=30.0)
    with pytest.raises(NotImplementedError):
        _impl(cls, attn_type=V.AttentionType.ENCODER)
    if cls is dsa.NPUDSAImpl:
        with pytest.raises(NotImplementedError):
            _impl(cls, sliding_window=128)
    else:
        # the MLA backend takes a window for its static-sink variant (reference mla.py:281) and keeps no sink by default
        impl = _impl(cls, sliding_window=128)
        assert impl.sliding_window == 128 and impl.sink_len == 0 and impl.sink_compressed_kv is None
        with pytest.raises(ValueError, match="sliding_window"):
            _impl(cls, sliding_window=0)


def test_update_sink_kv_and_sink_metadata():
    """update_sink_kv keeps the latents as the reference does (mla.py:304-307); the builder marks decode metadata with
    the sink length of the cache spec (mla.py:152-153)."""
    impl = _impl(mla.NPUMLAImpl)
    impl.update_sink_kv(torch.zeros(128, 64), torch.zeros(128, 512))
    assert impl.sink_len == 128 and impl.sink_k_pe.shape == (128, 1, 64) and impl.sink_compressed_kv.shape == (128, 512)
    spec = V.AttentionSpec(128, 1, 576, torch.bfloat16)
    spec.sink_len = 128
    builder = mla.NPUMLAMetadataBuilder(spec, ["l0"], _cfg(), torch.device("cpu"))
    md = builder.build(0, _common([1, 1, 1], [10, 200, 31]))
    assert md.decode.seq_sink_len == [128, 128, 128]
    md0 = mla.NPUMLAMetadataBuilder(V.AttentionSpec(128, 1, 576, torch.bfloat16), ["l0"], _cfg(), torch.device("cpu")).build(
        0, _common([1, 1], [10, 20]))
    assert md0.decode.seq_sink_len is None


@pytest.mark.parametrize("cls", [mla.NPUMLAImpl, dsa.NPUDSAImpl])
def test_impl_profile_run_and_argument_errors(cls):
    impl = _impl(cls)
    q, kc, kpe = torch.zeros(3, 8, 192), torch.zeros(3, 512), torch.zeros(3, 1, 64)
    out = torch.ones(5, 8 * 128)
    with pytest.raises(AssertionError, match="Output tensor must be provided"):
        impl.forward(None, q, kc, kpe, (), None, output=None)
    with pytest.raises(NotImplementedError, match="fused output quantization"):
        impl.forward(None, q, kc, kpe, (), None, output=out, output_scale=torch.ones(1))
    res = impl.forward(None, q, kc, kpe, (), None, output=out)          # attn_metadata is None: the profile run
    assert res is out and (out == 0).all()
    meta = SimpleNamespace(num_actual_tokens=3, num_decodes=0, num_prefills=0, num_decode_tokens=0)
    with pytest.raises(AssertionError):
        impl.forward(None, q, kc, kpe, (torch.zeros(1),), meta, output=out)   # wrong cache tuple arity


def test_v_up_proj_identity_known_answer():
    """Reference KAT, tests/unit/attention/backends/test_mla.py:190-259 (CPU tensors: the projection is a library bmm)."""
    n, bsz, vd = 32, 2, 128
    impl = _impl(mla.NPUMLAImpl, num_heads=n)
    x = torch.randn(n * bsz, 512, generator=torch.Generator().manual_seed(0)).bfloat16()
    impl.W_UV = torch.zeros(n, 512, vd, dtype=torch.bfloat16)
    for h in range(n):
        impl.W_UV[h, :vd, :] = torch.eye(vd, dtype=torch.bfloat16)
    out = impl._v_up_proj(x)
    expected = torch.zeros(bsz, n * vd, dtype=torch.bfloat16)
    for b in range(bsz):
        for h in range(n):
            expected[b, h * vd:(h + 1) * vd] = x[h * bsz + b, :vd]
    assert torch.allclose(out, expected, atol=1e-3)


def test_process_weights_after_loading_layout():
    """W_UK_T [N,P,L], W_UV [N,L,V] from kv_b_proj viewed [L, N, P+V] (test_npu_mla_math.py:302-313)."""
    n = 4
    lin = torch.nn.Linear(512, n * 256, bias=False)
    impl = _impl(mla.NPUMLAImpl, num_heads=n, kv_b_proj=lin)
    impl.process_weights_after_loading(torch.float32)
    w = lin.weight.t().reshape(512, n, 256)
    assert torch.equal(impl.W_UK_T, w[..., :128].permute(1, 2, 0)) and torch.equal(impl.W_UV, w[..., 128:].transpose(0, 1))


def test_kv_up_projection_goes_fp16_only_for_a_plain_weight():
    """_kv_up (reference: ``self.kv_b_proj(kv_c_normed)[0]``, mla.py:405-413) hands the prefill kernel fp16 keys and values
    when it is allowed to, the projection is a plain bf16 weight without bias and the switch is on; otherwise it calls the
    module.  Either way the numbers are the module's, up to the rounding of the result."""
    n = 2
    lin = torch.nn.Linear(512, n * 256, bias=False).to(torch.bfloat16)
    impl = _impl(mla.NPUMLAImpl, num_heads=n, kv_b_proj=lin)
    x = torch.randn(5, 512, generator=torch.Generator().manual_seed(1)).bfloat16()
    k16, v16 = impl._kv_up(x, allow_fp16=True)
    k, v = impl._kv_up(x)
    assert k16.dtype == v16.dtype == torch.float16 and k.dtype == v.dtype == torch.bfloat16
    assert k16.shape == k.shape == (5, n, 128) and v16.shape == v.shape == (5, n, 128)
    ref = (x.float() @ lin.weight.float().t()).view(5, n, 256)
    assert torch.allclose(k16.float(), ref[..., :128], atol=2e-3, rtol=2e-3) and torch.allclose(v16.float(), ref[..., 128:], atol=2e-3, rtol=2e-3)
    assert torch.allclose(k.float(), ref[..., :128], atol=2e-2, rtol=2e-2)
    impl.prefill_kv_fp16 = False
    assert impl._kv_up(x, allow_fp16=True)[0].dtype == torch.bfloat16
    impl.prefill_kv_fp16 = True
    impl.kv_b_proj = lambda t: (lin(t),)                       # no weight to be seen: the module is called
    assert impl._kv_up(x, allow_fp16=True)[0].dtype == torch.bfloat16
    biased = torch.nn.Linear(512, n * 256, bias=True).to(torch.bfloat16)
    impl.kv_b_proj = biased
    assert impl._kv_up(x, allow_fp16=True)[0].dtype == torch.bfloat16


# ---- graph wrapper (no GPU: pass-through paths only) ---------------------------------------------------------------
def test_graph_wrapper_pass_through_and_pad_list():
    calls = []
    runnable = lambda x: calls.append(x) or x + 1
    runnable_obj = SimpleNamespace(__call__=runnable, extra=7)
    w = HIPGraphWrapper(runnable, _cfg(), V.CUDAGraphMode.FULL)
    assert ACLGraphWrapper is HIPGraphWrapper and w.unwrap() is runnable
    with V.set_forward_context(None, V.BatchDescriptor(4), V.CUDAGraphMode.NONE):
        assert w(1) == 2                                      # NONE: eager
    with V.set_forward_context(None, V.BatchDescriptor(4), V.CUDAGraphMode.PIECEWISE):
        assert w(2) == 3                                      # another wrapper's mode: eager
    assert calls == [1, 2] and w.concrete_graph_entries == {}
    with pytest.raises(AssertionError):
        HIPGraphWrapper(runnable, _cfg(), V.CUDAGraphMode.NONE)
    assert w._pad_list([1, 2], 4) == [1, 2, 2, 2] and w._pad_list([1, 2], 4, 0) == [1, 2, 0, 0]
    assert w._pad_list([1, 2, 3], 2) == [1, 2] and w._pad_list([], 3) == [] and w._pad_list([5], 1) == [5]
    w2 = HIPGraphWrapper(SimpleNamespace(extra=7), _cfg(), V.CUDAGraphMode.FULL)
    assert w2.extra == 7
    with pytest.raises(AttributeError):
        w2.missing


def test_default_split_count_is_a_function_of_shapes_only():
    """About one chunk per compute unit, never fewer than eight 32-key blocks per chunk, at most 256 chunks per sequence;
    shapes of the benchmark configurations keep the counts they were measured with."""
    from omni_npu_amd import kernels as K
    assert K.default_num_splits(64, 1, 128, 8192) == 4            # headline: 256 chunks
    assert K.default_num_splits(32, 1, 128, 2048) == 8            # sparse decode over top-2048
    assert K.default_num_splits(256, 2, 128, 32768) == 1          # fp8 configuration: two row groups per sequence already
    assert K.default_num_splits(1, 1, 128, 131072) == 256         # one long sequence fills the device
    assert K.default_num_splits(1, 1, 128, 1000) == 4             # ... but a chunk keeps eight blocks
    assert K.default_num_splits(1, 1, 16, 1) == 1
    assert K.default_num_splits(4, 3, 128, 65536) == 22           # 4 x 3 row groups: ceil(256 / 12)
    for b in (1, 3, 64, 1000):
        for l in (1, 255, 256, 257, 10 ** 6):
            s = K.default_num_splits(b, 1, 128, l)
            assert 1 <= s <= 256 and (s == 1 or l / s >= 128)


# ---- the custom-model modules: routing (reference tests/unit/layers/test_npu_dsa.py:242-295) -----------------------
def _custom_module(cls, **extra):
    norm = SimpleNamespace(weight=torch.ones(512), variance_epsilon=1e-6)
    attn = SimpleNamespace(layer_name="model.layers.3.self_attn.attn", impl=None, kv_cache=[None])
    lin = lambda x: (x, None)
    return cls(256, 16, 128, 64, 128, 128, 512, attn, *extra.values(), lin, lin, lin, lin, norm, lin,
               prefix="model.layers.3.self_attn"), attn


def test_custom_model_mla_module_routes_by_metadata(monkeypatch):
    from omni_npu_amd.v1.layers.attention import NPUDeepseekMLAAttention
    mod, attn = _custom_module(NPUDeepseekMLAAttention)
    seen = []
    monkeypatch.setattr(mod, "_forward_prefill", lambda h, c, s, ctx, meta: seen.append(("prefill", meta)) or "p")
    monkeypatch.setattr(mod, "_forward_decode", lambda h, c, s, ctx, meta: seen.append(("decode", meta)) or "d")
    x = torch.zeros(2, 256)
    with V.set_forward_context(attn_metadata=None):                                    # profile run -> prefill branch
        assert mod(x, None, None) == "p" and seen[-1] == ("prefill", None)
    pre = SimpleNamespace(prefill=object(), decode=None)
    dec = SimpleNamespace(prefill=None, decode=object())
    with V.set_forward_context(attn_metadata={attn.layer_name: pre, "other": dec}):     # dict: looked up by layer name
        assert mod(x, None, None) == "p" and seen[-1] == ("prefill", pre)
    with V.set_forward_context(attn_metadata=dec):
        assert mod(x, None, None) == "d" and seen[-1] == ("decode", dec)
    with V.set_forward_context(attn_metadata=SimpleNamespace(prefill=object(), decode=object())):
        with pytest.raises(NotImplementedError):
            mod(x, None, None)


def test_custom_model_modules_need_a_norm_with_parameters():
    from omni_npu_amd.v1.layers.attention import NPUDeepseekMLAAttention, NPUDeepseekSparseAttention
    lin = lambda x: (x, None)
    attn = SimpleNamespace(layer_name="l", impl=None, kv_cache=[None])
    with pytest.raises(TypeError):
        NPUDeepseekMLAAttention(256, 16, 128, 64, 128, 128, 512, attn, lin, lin, lin, lin, lambda v: v, lin)
    with pytest.raises(TypeError):
        NPUDeepseekSparseAttention(256, 16, 128, 64, 128, 128, 512, attn, None, lin, lin, lin, lin, lambda v: v, lin)
    mod = NPUDeepseekSparseAttention(256, 16, 128, 64, 128, 128, 512, attn, None, lin, lin, lin, lin,
                                     SimpleNamespace(weight=torch.ones(512), eps=1e-6), lin)
    with V.set_forward_context(attn_metadata=SimpleNamespace(prefill=object(), decode=object())):
        with pytest.raises(NotImplementedError):
            mod(torch.zeros(2, 256), None, None)


def test_workspace_growth_keeps_the_retained_scratch_bounded():
    """Scratch buffers are never freed (captured graphs hold their addresses); the growth rule bounds what a key retains:
    at most 2 + log1.5(max / first) buffers and less than 4.5 x the largest request in total."""
    import math
    import random
    from omni_npu_amd import kernels as K
    rng = random.Random(0)
    for trial in range(200):
        reqs = [rng.randint(64, 1 << rng.randint(7, 30)) for _ in range(rng.randint(1, 60))]
        sizes, have = [], 0
        for r in reqs:
            new = K._workspace_growth(have, r)
            if new:
                assert new >= r and new >= (have * 3) // 2
                sizes.append(new)
                have = new
            assert have >= r
        m = max(reqs)
        assert len(sizes) <= 2 + math.log(m / sizes[0]) / math.log(1.49)
        assert sum(sizes) < 4.5 * m + len(sizes)
    assert K._workspace_growth(100, 100) == 0 and K._workspace_growth(0, 0) == 1 and K._workspace_growth(100, 101) == 150


def test_builder_keeps_widened_seq_lens_in_one_int32_buffer():
    """A runner that hands over int64 lengths (the reference widens them, npu_model_runner.py:81-86) must not give every
    step a fresh int32 tensor: a graph captured over one step would read stale lengths.  int32 input passes through."""
    spec = V.AttentionSpec(128, 1, 576, torch.bfloat16)
    for builder in (mla.NPUMLAMetadataBuilder(spec, ["l0"], _cfg(cap=4), torch.device("cpu")),
                    dsa.NPUDSAMetadataBuilder(spec, ["l0"], _cfg(cap=4), torch.device("cpu"))):
        c = _common([1, 1, 1], [300, 130, 2])
        assert builder.build(0, c).decode.seq_lens.data_ptr() == c.seq_lens.data_ptr()
        ptrs = []
        for lens in ([300, 130, 2], [301, 131, 3], [5, 6, 7]):
            c = _common([1, 1, 1], lens)
            c.seq_lens = c.seq_lens.to(torch.int64)
            d = builder.build(0, c).decode
            assert d.seq_lens.dtype == torch.int32 and d.seq_lens.tolist() == lens
            ptrs.append(d.seq_lens.data_ptr())
        assert len(set(ptrs)) == 1
