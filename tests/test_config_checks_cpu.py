"""The configuration checks of tests/config_checks.py on the CPU operator package at reduced sizes: the same
functions the GPU tests run at the configurations' full sizes, so this also proves the checks themselves."""
import torch

import config_checks as cc


def test_dense_with_downstream_on_the_cpu_package():
    import l1attn_cpp
    errs = cc.dense_with_downstream(l1attn_cpp, torch.device("cpu"), 3, 96, 4, 32)
    assert errs[0] <= cc.FWD_TOL and errs[1] <= cc.FWD_TOL and errs[2] <= cc.BWD_TOL and errs[3] <= cc.BWD_TOL


def test_sparse_uniform_graph_on_the_cpu_package():
    import l1attn_sparse_cpp
    E, errs = cc.sparse_uniform_graph(l1attn_sparse_cpp, torch.device("cpu"), 2, 256, 4, 32, max_deg=16)
    assert 256 <= E <= 256 * 16
    assert errs[0] <= cc.FWD_TOL and max(errs[1:]) <= cc.BWD_TOL


def test_bidi_powerlaw_graph_on_the_cpu_package():
    import l1attn_sparse_bidi_cpp
    E, dmx, errs = cc.bidi_powerlaw_graph(l1attn_sparse_bidi_cpp, torch.device("cpu"), 1, 2048, 2, 64)
    assert E > 2 * 2048 and dmx > 128            # long segments are part of the case
    assert errs[0] <= cc.FWD_TOL and max(errs[1:]) <= cc.BWD_TOL


def test_dense_sampled_rows_on_the_cpu_package():
    import _l1attn_cpu
    for layernorm in (False, True):
        errs = cc.dense_sampled_rows(_l1attn_cpu, torch.device("cpu"), 2, 160, 4, 32, layernorm,
                                     [(0, 0), (1, 159), (1, 77)])
        assert errs[0] <= cc.FWD_TOL and errs[1] <= cc.BWD_TOL and errs[2] <= cc.BWD_TOL and errs[3] <= 1e-4
