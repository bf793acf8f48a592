"""The importance-weighted search of the oracle, pinned by the reference's own property tests
(tests/llmcompressor/observers/test_imatrix.py:217-268) and by a brute-force argmin in fp64."""
import torch

from oracle import observers as O
from oracle.qformat import QArgs, calculate_qparams, fake_quantize


def _observed(w, args):
    return O.flatten_for_calibration(w, "weight", args)


def test_uniform_importance_matches_plain_search_on_fp32():
    """test_imatrix.py:239-268: all-ones importance, norm 2.4, maxshrink 0.2, grid 20 gives the scales of
    memoryless_mse with grid 20 (fp32 weights: both searches then form the error in fp32)."""
    torch.manual_seed(123)
    w = torch.nn.Linear(8, 4).weight.detach()
    args = QArgs(num_bits=4, symmetric=True, strategy="channel")
    obs = _observed(w, args)
    imp = O.prepare_importance(torch.ones(8), 1, obs, args)
    mn_i, mx_i = O.imatrix_grid_search(obs, args, maxshrink=0.20, grid=20, norm=2.4, importance_weights=imp)
    mn_u, mx_u = O.grid_search_mse(obs, args, maxshrink=0.20, grid=20, norm=2.4)
    s_i, z_i = calculate_qparams(mn_i, mx_i, args)
    s_u, z_u = calculate_qparams(mn_u, mx_u, args)
    assert torch.allclose(s_i, s_u) and torch.equal(z_i, z_u)


def test_importance_changes_result():
    """test_imatrix.py:217-237"""
    torch.manual_seed(123)
    w = torch.nn.Linear(8, 4).weight.detach()
    args = QArgs(num_bits=4, symmetric=True, strategy="channel")
    obs = _observed(w, args)
    imp = O.prepare_importance(torch.tensor([1000.0] * 4 + [0.01] * 4), 1, obs, args)
    a = O.imatrix_grid_search(obs, args, importance_weights=imp)
    b = O.imatrix_grid_search(obs, args)
    assert not torch.allclose(calculate_qparams(*a, args)[0], calculate_qparams(*b, args)[0])


def test_matches_brute_force_argmin_in_fp64():
    """Every group's chosen range is the first candidate attaining the smallest weighted error (patience 0)."""
    g = torch.Generator().manual_seed(7)
    w = torch.randn(6, 64, generator=g)
    imp_raw = torch.rand(64, generator=g) * 5 + 0.01
    for args in (QArgs(num_bits=4, symmetric=True, strategy="group", group_size=16),
                 QArgs(num_bits=4, symmetric=False, strategy="channel")):
        obs = _observed(w, args)
        imp = O.prepare_importance(imp_raw, 1, obs, args)
        mn, mx = O.imatrix_grid_search(obs, args, patience=0, importance_weights=imp)
        token = args.copy(strategy="token")
        mn0, mx0 = torch.amin(obs, dim=(0, -1)), torch.amax(obs, dim=(0, -1))
        errs = []
        for i in range(int(0.95 * 20) + 1):
            p = 1 - i / 20
            s, z = calculate_qparams(p * mn0, p * mx0, args)
            q = fake_quantize(obs, s.unsqueeze(-1), z.unsqueeze(-1), token)
            errs.append(((q.double() - obs.double()).abs() ** 3 * imp.double()).sum(dim=(0, -1)))
        errs = torch.stack(errs)  # [candidates, *groups]
        best = errs.argmin(0)
        p_best = 1 - best.float() / 20
        close = torch.isclose(mn, p_best * mn0) & torch.isclose(mx, p_best * mx0)
        # fp32 vs fp64 sums may swap two candidates whose errors agree to 1e-6
        chosen = torch.zeros_like(best)
        for i in range(errs.shape[0]):
            chosen = torch.where(torch.isclose(mn, (1 - i / 20) * mn0) & torch.isclose(mx, (1 - i / 20) * mx0) & (chosen == 0),
                                 torch.full_like(best, i), chosen)
        gap = (errs.gather(0, chosen.unsqueeze(0))[0] - errs.min(0)[0]) / errs.min(0)[0]
        assert bool((close | (gap < 1e-5)).all())


def test_patience_semantics():
    """patience > 0 stops the whole search after that many candidates without any improvement; 0 never stops."""
    w = torch.tensor([[0.0, 1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0]])  # exactly representable at p = 1: error 0
    args = QArgs(num_bits=4, symmetric=False, strategy="channel")
    obs = _observed(w, args)
    mn, mx = O.imatrix_grid_search(obs, args, patience=1)
    assert float(mx) == 7.0 and float(mn) == 0.0
