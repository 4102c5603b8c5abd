"""Sampling kernels (GPU)."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("V", [7001, 73448, 20000, 36])       # odd (one logit a load) and multiples of 4 (four)
def test_argmax_ties_go_to_the_lowest_index(V):
    from cpmcu_amd import ops
    lg = torch.randn(5, V, generator=torch.Generator().manual_seed(0)).to(DEV)
    lg[1, V - 1001 if V > 2000 else V - 3] = lg[1, 17] = 50.0
    lg[2, 0] = 60.0
    lg[3, V - 1] = 60.0
    lg[4, V // 2 + 1] = lg[4, V // 2 + 2] = 70.0
    out = torch.empty(5, dtype=torch.int32, device=DEV)
    ops.argmax(lg, out)
    want = lg.argmax(-1).tolist()
    want[1] = 17
    want[4] = V // 2 + 1
    assert out.tolist() == want


def test_draws_follow_softmax_and_do_not_depend_on_the_batch():
    from cpmcu_amd import ops
    from cpmcu_amd.sampling import Sampler
    V, N = 37, 20000
    row = torch.randn(V, generator=torch.Generator().manual_seed(1)) * 2
    lg = row.repeat(N, 1).to(DEV).contiguous()
    temp = 0.8
    s = Sampler(temp, seed=1234)
    toks = s.sample(lg, list(range(N)), [0] * N)
    freq = torch.bincount(toks.long().cpu(), minlength=V).double()
    p = torch.softmax(row.double() / temp, 0)
    chi2 = float(((freq - N * p) ** 2 / (N * p)).sum())
    assert chi2 < 80, chi2                                  # 36 degrees of freedom: P(chi2 > 80) < 1e-4
    # the same (seed, request, step) draws the same token whatever else is in the batch
    again = s.sample(lg[:10], [5, 3, 9, 5, 100, 7, 8, 0, 1, 2], [0] * 10)
    assert again.tolist() == [int(toks[i]) for i in [5, 3, 9, 5, 100, 7, 8, 0, 1, 2]]
    other_step = s.sample(lg[:64], list(range(64)), [1] * 64)
    assert other_step.tolist() != toks[:64].tolist()
    assert Sampler(temp, seed=99).sample(lg[:64], list(range(64)), [0] * 64).tolist() != toks[:64].tolist()
    # a very low temperature is greedy; temperature 0 takes the argmax kernel
    cold = Sampler(1e-4, seed=5).sample(lg[:8], list(range(8)), [0] * 8)
    assert cold.tolist() == [int(row.argmax())] * 8
    assert Sampler(0.0).sample(lg[:8], list(range(8)), [0] * 8).tolist() == [int(row.argmax())] * 8
    with pytest.raises(ops.KernelError, match="temperature"):
        ops.sample(lg[:1], 0.0, 1, torch.zeros(1, dtype=torch.int32, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV),
                   torch.zeros(1, dtype=torch.int32, device=DEV))


def test_a_large_vocabulary_row_with_one_dominant_token():
    from cpmcu_amd.sampling import Sampler
    V = 73448
    lg = torch.zeros(3, V, device=DEV)
    lg[:, 70001] = 40.0
    assert Sampler(1.0, seed=3).sample(lg, [0, 1, 2], [0, 0, 0]).tolist() == [70001] * 3
