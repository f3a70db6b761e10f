"""The example self-checks (the reference's own acceptance style: PCC > 0.97 against torch) run as a test,
plus the definition of torch_pcc on its corner cases."""
import math

import pytest
import torch

from triton_tenstorrent_amd.examples import validate as V


def test_torch_pcc_definition():
    a = torch.tensor([1.0, 2.0, 3.0, 4.0])
    assert math.isclose(V.torch_pcc(a, 2 * a + 1), 1.0, rel_tol=1e-12)
    assert math.isclose(V.torch_pcc(a, -a), -1.0, rel_tol=1e-12)
    x = torch.tensor([1.0, 2.0, 4.0, 7.0])
    y = torch.tensor([1.5, 1.0, 5.0, 6.0])
    assert math.isclose(V.torch_pcc(x, y), float(torch.corrcoef(torch.stack([x, y]))[0, 1]), rel_tol=1e-6)
    # non-finite positions are dropped on both sides
    assert math.isclose(V.torch_pcc(torch.tensor([1.0, float("nan"), 3.0, 5.0]), torch.tensor([2.0, 9.0, 6.0, 10.0])), 1.0,
                        rel_tol=1e-12)
    # degenerate: constant vectors, one value
    assert V.torch_pcc(torch.ones(5), torch.ones(5)) == 1.0 and V.torch_pcc(torch.ones(5), torch.zeros(5)) == 0.0
    assert V.torch_pcc(torch.tensor([3.0]), torch.tensor([3.0])) == 1.0


@pytest.mark.gpu
def test_examples_meet_the_references_bar(capsys):
    torch.manual_seed(0)
    assert V.main() == 0
    out = capsys.readouterr().out
    assert out.count("PCC = ") == 12 and out.rstrip().endswith("Success!")
    # far inside the 0.97 bar: these kernels are not bf16-on-a-different-device approximations
    assert V.validate_matmul(64, 32, 64, verbose=False) > 0.9999
    assert V.validate_sin(1024, verbose=False) > 0.999999
