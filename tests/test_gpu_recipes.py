"""The benchmark configurations on their own seeded recipes, at full size: the rank the fit returns and the relative
residual of the basis it hands out, against what the recipe fixes in closed form (bench.recipe_expectation: the energy
rule of src/gram_evd.cu:58-60 on the recipe's singular values and noise level; for the interpolation the stopping rule of
src/hyacin_potrfp.cu:224-269).  The bar is the path's: rank within one, residual within twice the expected one."""
import ctypes as C

import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg3", "cfg4", "cfg4seg", "cfg5", "target"])
def test_fit_on_the_recipe_of_the_configuration(name):
    import torch
    import bench
    import hyacinth_amd as ha
    L = ha.lib()
    num, at, opA, M, N, K, eps, alg, fit_name, desc = bench.WORKLOADS[name]
    cplx = at & 1
    print("recipe", name, desc, flush=True)
    torch.cuda.empty_cache()
    h = ha.create_handle(stream=torch.cuda.current_stream().cuda_stream, GramMatrixAlgorithm=alg)
    try:
        A, lda = bench.make_workload(torch, name)
        real = torch.float64 if at in (0, 1) else (torch.float32 if at in (2, 3) else torch.float16)
        S = torch.zeros(max(K, N), dtype=torch.float64, device="cuda")
        V = torch.zeros(N * K * (2 if cplx else 1), dtype=real, device="cuda")
        rank = getattr(L, fit_name)(C.byref(h), eps, opA.encode(), M, N, K, C.c_void_p(A.data_ptr()), lda, C.c_void_p(S.data_ptr()), C.c_void_p(V.data_ptr()), N, 0, at)
        torch.cuda.synchronize()
        assert L.hykLastStatus() == 0 and rank > 0
        got = bench.fit_quality(torch, L, h, name, A, lda, rank, S, V)
        want = bench.recipe_expectation(name, rank)
        print("recipe", name, "rank", rank, "expected", want["expected_rank"], "relative residual", got, "expected", want["expected_rel_residual"], flush=True)
        if want["expected_rank"] is not None:
            assert abs(rank - want["expected_rank"]) <= 1
        else:
            assert rank <= K
        assert got <= 2.0 * want["expected_rel_residual"]
        if fit_name != "hyacinInterpolateFit":                   # singular values: the recipe's, to 10 eps of the largest (where the noise floor leaves them alone)
            Sh = S.view(real)[:K].double().cpu().numpy()
            assert (Sh[:rank] > 0).all() and (Sh[rank:] == 0).all() and (Sh[:rank - 1] >= Sh[1:rank]).all()
            closed = bench.recipe_values(name)
            if closed is not None:
                s, moved = closed
                storage_eps = {torch.float64: 2.2e-16, torch.float32: 6e-8, torch.float16: 4.9e-4}[real]
                worst = float(abs(Sh[:rank] - s[:rank]).max())
                print("recipe", name, "largest distance of a singular value from the recipe's", worst, "allowed", 10 * max(eps, storage_eps) * s[0] + moved, flush=True)
                assert worst <= 10 * max(eps, storage_eps) * s[0] + moved
    finally:
        ha.destroy_handle(h)
        del h
        torch.cuda.empty_cache()
