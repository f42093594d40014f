"""Workspace options that fix what the library otherwise picks from a workspace's history
(HOMCOMP_OPT_LDS_BUDGET, HOMCOMP_OPT_PLANE_PATHS) and the report of what a call was launched with
(homcomp_workspace_last_launch): every choice gives the oracle's bytes, the report names it."""
import numpy as np
import pytest

from gpu_util import Gpu, first_diff

pytestmark = pytest.mark.gpu


def test_fixed_budget_and_kernel_kind(pkg, cuda, orc, gen):
    orc.set_threads(16)
    n = (1 << 20) + 32768 * 3
    g = Gpu(pkg, cuda, n)
    try:
        assert g.ws.last_launch() == {"kernel": None, "lds_budget": None}
        a, b = gen.smooth_np(n, 71), gen.gradient_like_np(n, 72)
        eb = np.float32(2e-4)
        sa, sb = orc.compress(a, eb), orc.compress(b, eb)
        want_s, want_i = orc.hom_sum_f32(sa, b, eb), orc.hom_sum_i32(sa, orc.quant_predict(b, eb))
        want_add = orc.hom_add(sa, sb, n)
        qp = orc.quant_predict(b, eb)
        for budget, name in ((0, "small"), (1, "medium"), (2, "large"), (-1, None)):
            g.ws.set_option(pkg.OPT_LDS_BUDGET, budget)
            got = g.compress(a, eb)
            assert np.array_equal(got, sa), f"compress, budget {name}: {first_diff(got, sa)}"
            launched = g.ws.last_launch()
            assert launched["kernel"] == "general" and (name is None or launched["lds_budget"] == name)
            for paths, kinds in ((0, ("general", "general")), (2, ("few_planes", "few_planes")), (3, (None, "wide_planes")),
                                 (1, (None, None))):
                g.ws.set_option(pkg.OPT_PLANE_PATHS, paths)
                got = g.hom_sum_f32(sa, b, eb)
                assert np.array_equal(got, want_s), f"hom_sum_f32, budget {name}, paths {paths}: {first_diff(got, want_s)}"
                launched = g.ws.last_launch()
                assert kinds[0] is None or launched["kernel"] == kinds[0]
                assert name is None or launched["lds_budget"] == name
                got = g.hom_sum_i32(sa, qp)
                assert np.array_equal(got, want_i), f"hom_sum_i32, budget {name}, paths {paths}"
                got = g.hom_add(sa, sb, n)
                assert np.array_equal(got, want_add), f"hom_add, budget {name}, paths {paths}: {first_diff(got, want_add)}"
                assert kinds[1] is None or g.ws.last_launch()["kernel"] == kinds[1]
        L = pkg.lib()
        assert L.homcomp_workspace_set_option(g.ws._h, pkg.OPT_LDS_BUDGET, 3) == -1
        assert L.homcomp_workspace_set_option(g.ws._h, pkg.OPT_PLANE_PATHS, 4) == -1
        assert L.homcomp_workspace_last_launch(None, None, None) == -1
    finally:
        g.close()
