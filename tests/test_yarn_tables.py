"""YaRN-scaled rotary tables (reference layers/rotary_embedding/deepseek_scaling_rope.py:51-87).  The helper functions
the reference imports from vLLM are not in its tree, so the oracle restates the published formulation and is pinned here by
what the mathematics and the published DeepSeek-V3 configuration fix; the module is then checked against the oracle."""
import math

import pytest
import torch

from oracle import mla_oracle as O


def test_oracle_yarn_reduces_to_plain_tables_without_scaling():
    pos = torch.tensor([0, 1, 7, 100, 4095])
    c0, s0 = O.rope_tables(pos, dtype=torch.float32)
    c1, s1 = O.yarn_rope_tables(pos, scaling_factor=1.0, dtype=torch.float32)
    assert torch.allclose(c0, c1, atol=2e-4) and torch.allclose(s0, s1, atol=2e-4)   # (fp32 angles in the plain tables)


def test_oracle_yarn_known_constants_and_regimes():
    """DeepSeek-V3: 64 dims, base 1e4, factor 40 over 4096 positions, beta 32 / 1: the ramp runs over pairs 10..23;
    mscale = mscale_all_dim leaves the values unscaled; mscale 1 alone gives 0.1 ln 40 + 1."""
    d, base, f, L = 64, 10000.0, 40.0, 4096
    corr = lambda rot: d * math.log(L / (rot * 2 * math.pi)) / (2 * math.log(base))
    assert (math.floor(corr(32)), math.ceil(corr(1))) == (10, 23)
    pos = torch.tensor([1.0])
    c, s = O.yarn_rope_tables(pos, mscale=1.0, mscale_all_dim=1.0, dtype=torch.float64)
    ang = torch.atan2(s[0, :32], c[0, :32])                       # angle of pair i at position 1 = its frequency
    plain = torch.tensor([base ** (-2.0 * i / d) for i in range(32)], dtype=torch.float64)
    assert torch.allclose(ang[:11], plain[:11], rtol=1e-12)       # fast pairs: untouched
    assert torch.allclose(ang[23:], plain[23:] / f, rtol=1e-12)   # slow pairs: divided by the factor
    mid = ang[11:23] / plain[11:23]
    assert ((mid < 1) & (mid > 1 / f)).all() and (mid[1:] < mid[:-1]).all()   # a monotone blend in between
    assert torch.allclose((c ** 2 + s ** 2)[0], torch.ones(64, dtype=torch.float64))     # no scaling of the values
    c2, s2 = O.yarn_rope_tables(pos, mscale=1.0, mscale_all_dim=0.0, dtype=torch.float64)
    assert torch.allclose((c2 ** 2 + s2 ** 2)[0].sqrt(), torch.full((64,), 0.1 * math.log(40.0) + 1.0, dtype=torch.float64))
    assert torch.equal(c[:, :32], c[:, 32:]) and torch.equal(s[:, :32], s[:, 32:])       # rows are cat(c, c)


@pytest.mark.parametrize("kw", [dict(mscale=1.0, mscale_all_dim=1.0), dict(mscale=1.0, mscale_all_dim=0.0),
                                dict(mscale=0.707, mscale_all_dim=0.707, beta_fast=16, beta_slow=2, attn_factor=1.5)])
def test_module_tables_match_the_oracle(kw):
    from omni_npu_amd.layers.rotary_embedding import HIPDeepseekScalingRotaryEmbedding
    rot = HIPDeepseekScalingRotaryEmbedding(64, 64, 256, 10000.0, False, 40.0, torch.float32, **kw)
    assert rot.cos_cached.shape == (256 * 40, 64)                 # the table covers the extended context
    pos = torch.tensor([0, 1, 2, 63, 500, 4095, 10239])
    params = dict(kw, original_max_position=256)
    c, s = O.yarn_rope_tables(pos, scaling_factor=40.0, dtype=torch.float32, **params)
    gc, gs = rot.get_cos_sin(pos)
    # fp32 angles of up to 1e4 radians carry 1e-3 of absolute error; small positions agree to fp32 rounding
    assert torch.allclose(gc[:4], c[:4], atol=1e-5) and torch.allclose(gs[:4], s[:4], atol=1e-5)
    assert torch.allclose(gc, c, atol=2e-3) and torch.allclose(gs, s, atol=2e-3)
    with pytest.raises(NotImplementedError):
        HIPDeepseekScalingRotaryEmbedding(64, 64, 256, 10000.0, True, 40.0)
