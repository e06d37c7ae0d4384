"""Golden vectors of tests/golden/ (written by tests/golden/make_fixtures.py).

CPU: the oracle reproduces them (the oracle cannot drift unnoticed) and the two structured cases of the
reference's scripts have their closed-form values.  GPU: the HIP path, through the C ABI, matches the files.
"""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests._util import assert_close

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FILES = sorted(glob.glob(os.path.join(HERE, "*.npz")))
NAMES = [os.path.basename(f)[:-4] for f in FILES]


def _load(name):
    z = np.load(os.path.join(HERE, name + ".npz"), allow_pickle=False)
    x = {k[3:]: torch.from_numpy(z[k]) for k in z.files if k.startswith("in_")}
    y = {k[4:]: torch.from_numpy(z[k]) for k in z.files if k.startswith("out_")}
    return x, y


def test_fixture_files_are_present():
    assert set(NAMES) >= {"seeded_small", "seeded_pooled_oddC", "seeded_c256", "ones_c10", "debug_bwd"}


@pytest.mark.parametrize("name", NAMES)
def test_oracle_reproduces_the_golden_vectors(name):
    x, y = _load(name)
    d = {k: (v if v.dtype == torch.int32 else v.double()) for k, v in x.items()}
    out_u, out_v, am_u, am_v = O.max_argmax_avg_forward(d["f1"], d["f2"])
    cu, cv = O.compression_forward(d["f1"], d["f2"], d["a_u"], d["a_v"])
    m1, m2 = O.max_argmax_avg_backward(d["f1"], d["f2"], d.get("am_u", am_u), d.get("am_v", am_v), d["g_u"], d["g_v"])
    c1, c2, da_u, da_v = O.compression_backward(d["f1"], d["f2"], d["a_u"], d["a_v"], d["g_cu"], d["g_cv"])
    got = dict(out_u=out_u, out_v=out_v, comp_u=cu, comp_v=cv, m_df1=m1, m_df2=m2, c_df1=c1, c_df2=c2, da_u=da_u, da_v=da_v)
    for k, v in got.items():
        assert torch.allclose(v.float(), y[k], rtol=1e-6, atol=1e-6), k
    assert torch.equal(am_u, y["am_u"]) and torch.equal(am_v, y["am_v"])


def test_structured_cases_have_their_closed_forms():
    _, y = _load("ones_c10")      # S = 10 everywhere; sums over 8 columns and 4 rows of weight 1
    assert torch.all(y["comp_u"] == 80) and torch.all(y["comp_v"] == 40)
    assert torch.all(y["out_u"] == 10) and torch.all(y["out_v"] == 10) and torch.all(y["am_u"] == 0)
    x, y = _load("debug_bwd")     # f = 1: d_f1 = sum over (u,v) of G, the same for every channel
    g = torch.arange(15.)
    # per row u the max term hits one column and the avg term is W * (u / W); the same for the columns
    expect = (g.sum() + g.sum()) + (g.sum() + g.sum())
    assert torch.allclose(y["m_df1"], torch.full_like(y["m_df1"], float(expect)))


@pytest.mark.gpu
@pytest.mark.parametrize("name", NAMES)
def test_hip_path_matches_the_golden_vectors(device, name):
    from separableflowthesis_amd import MemorySaver as ms
    x, y = _load(name)
    d = {k: v.to(device) for k, v in x.items()}
    out_u, out_v, am_u, am_v = ms.max_argmax_avg_forward(d["f1"], d["f2"])
    assert_close(out_u, y["out_u"], "max_avg_output_u")
    assert_close(out_v, y["out_v"], "max_avg_output_v")
    if name != "debug_bwd":   # all-ones volumes tie everywhere: index 0 by the lowest-index rule, as stored
        assert torch.equal(am_u.cpu(), y["am_u"]) and torch.equal(am_v.cpu(), y["am_v"])
    cu, cv = ms.compression_forward(d["f1"], d["f2"], d["a_u"], d["a_v"])
    assert_close(cu, y["comp_u"], "compression_output_u")
    assert_close(cv, y["comp_v"], "compression_output_v")
    m1, m2 = ms.max_argmax_avg_backward(d["f1"], d["f2"], d.get("am_u", am_u), d.get("am_v", am_v), d["g_u"], d["g_v"])
    assert_close(m1, y["m_df1"], "grad_fmap1_l0 (max/avg)", scale_atol=True)
    assert_close(m2, y["m_df2"], "grad_fmap2_lk (max/avg)", scale_atol=True)
    c1, c2, da_u, da_v = ms.compression_backward(d["f1"], d["f2"], d["a_u"], d["a_v"], d["g_cu"], d["g_cv"])
    for got, key in ((c1, "c_df1"), (c2, "c_df2"), (da_u, "da_u"), (da_v, "da_v")):
        assert_close(got, y[key], key, scale_atol=True)
    f1, f2 = ms.fused_backward(d["f1"], d["f2"], d.get("am_u", am_u), d.get("am_v", am_v), d["g_u"], d["g_v"],
                               d["a_u"], d["a_v"], d["g_cu"], d["g_cv"])
    assert_close(f1, y["m_df1"] + y["c_df1"], "fused grad_fmap1_l0", scale_atol=True)
    assert_close(f2, y["m_df2"] + y["c_df2"], "fused grad_fmap2_lk", scale_atol=True)
