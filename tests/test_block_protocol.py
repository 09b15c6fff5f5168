"""How a block hands a norm's input on (no GPU: the parts here are stand-ins that record calls)."""
import torch

from rbitnet_amd.parts.block import normed_for
from rbitnet_amd.parts.norm import GainedRows


class _Env:
    dtype = torch.bfloat16


class _Norm:
    folds_into_products = True

    def __init__(self):
        self.size, self.eps, self.env, self.weight = 4, 1e-5, _Env(), torch.ones(4)
        self.calls = []

    def forward(self, x, delta=None, rows=None):
        self.calls.append((delta, rows))
        return "normalised"


class _Takes:
    takes_gained_rows = True


class _Plain:
    pass


def _gained(norm, x):
    return GainedRows(norm, x, torch.zeros(3, 4, dtype=torch.bfloat16), torch.zeros(3, 1))


def test_gained_rows_go_on_only_to_their_norm_and_to_a_part_that_takes_them():
    x = torch.zeros(3, 4)
    norm, other = _Norm(), _Norm()
    left = _gained(norm, x)
    assert normed_for(_Takes(), norm, x, left) is left
    assert norm.calls == []
    # a part that wants a tensor, or another norm: the stream already holds the sum, so nothing is added
    assert normed_for(_Plain(), norm, x, left) == "normalised"
    assert norm.calls == [(None, None)]
    assert normed_for(_Takes(), other, x, left) == "normalised"
    assert other.calls == [(None, None)]


def test_pending_tensor_and_nothing_pending_are_normalised_by_the_norm():
    x = torch.zeros(3, 4)
    norm = _Norm()
    delta = torch.ones(3, 4)
    assert normed_for(_Takes(), norm, x, delta) == "normalised"
    assert normed_for(_Takes(), norm, x, None) == "normalised"
    assert norm.calls[0][0] is delta and norm.calls[1][0] is None


def test_rows_are_chosen_once():
    x = torch.zeros(3, 4)
    norm = _Norm()
    rows = torch.tensor([2, 0], dtype=torch.int32)
    picked = normed_for(_Takes(), norm, x, _gained(norm, x), rows)
    assert picked.rows is rows and picked.shape == (2, 4) and picked.gained.shape == (3, 4)
    assert picked.tensor() == "normalised" and norm.calls == [(None, rows)]
