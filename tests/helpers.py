"""Shared helpers for the test-suite: error metrics with the tolerances the parity bar names, fixture loading."""
import os

import numpy as np
import torch

from oracle import d2dmoe_oracle as O
from tests.golden import make_fixtures as MF

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')

# Parity bar for layer outputs: relative error (max |got - want| / max |want|) against the float64 evaluation of
# the oracle on the same stored inputs.
TOL_F32 = 1e-5
TOL_BF16 = 2e-2
TOL_F16 = 4e-3     # float16 keeps 11 significant bits where bfloat16 keeps 8


class GELUTanh(torch.nn.GELU):
    """An activation class of its own for the tanh form of GELU, as transformers has for Gemma (the layer and the surgery
    rebuild an activation from its type alone, moefication.py:116)."""

    def __init__(self):
        super().__init__(approximate='tanh')


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    denom = want.abs().max().item()
    if denom == 0.0:
        return got.abs().max().item()
    return (got - want).abs().max().item() / denom


def elem_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Element-wise companion of rel_err: max |got - want| / (|want| + max|want| / 8).  Unlike the max-norm ratio it
    holds every element to a bound that shrinks with the element, down to a floor of an eighth of the largest one: an
    output is a sum over ~2400 hidden activations that are each rounded to 16 bits (as the reference's own intermediate
    is), so the absolute error of a small element is that of a large one -- measured 1.4e-3 * max|want| on the GPT-2 layer
    in bfloat16, which a floor of a sixteenth would put at 2.2e-2."""
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    floor = want.abs().max().item() / 8.0
    if floor == 0.0:
        return got.abs().max().item()
    return ((got - want).abs() / (want.abs() + floor)).max().item()


def tol_for(dtype) -> float:
    return {torch.float32: TOL_F32, torch.bfloat16: TOL_BF16, torch.float16: TOL_F16}[dtype]


def load_fixture(name):
    return np.load(os.path.join(GOLDEN, f'{name}.npz'), allow_pickle=False)


def fixture_inputs(name, dtype):
    """Regenerates a fixture's inputs from its seed and verifies them against the stored checksum."""
    fx = load_fixture(name)
    x, p = MF.make_inputs(name, dtype)
    key = 'checksum_f32' if dtype == torch.float32 else 'checksum_bf16'
    assert MF.inputs_checksum(x, p) == str(fx[key]), f'fixture {name}: regenerated inputs differ from the stored ones'
    return fx, x, p, MF.CASES[name]


def routing_from_bits(bits: np.ndarray, n_experts: int) -> torch.Tensor:
    return torch.from_numpy(np.unpackbits(bits, axis=1)[:, :n_experts].astype(np.float32))


def random_case(N, D, E, Ed, W, seed, dtype, gated=False, bias=True, density=0.5, device='cpu'):
    p = O.make_layer_params(D, E, Ed, W, seed=seed, gated=gated, bias=bias, dtype=dtype)
    g = torch.Generator().manual_seed(seed + 99)
    x = torch.randn(N, D, generator=g).to(dtype)
    routing = (torch.rand(N, E, generator=g) < density).to(dtype)
    if 'last_bias' in p:
        p['last_bias'] = (torch.randn(1, D, generator=g) * 0.05).to(dtype)
    if device != 'cpu':
        x, routing = x.to(device), routing.to(device)
        p = {k: v.to(device) for k, v in p.items()}
    return x, routing, p


def to_dev(p, device):
    return {k: v.to(device) for k, v in p.items()}
