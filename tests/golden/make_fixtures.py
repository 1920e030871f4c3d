"""Writes the golden fixtures under tests/golden/ from the CPU oracle (oracle/d2dmoe_oracle.py) alone.

    python tests/golden/make_fixtures.py

The reference repository holds no golden vectors for the MoE forward path, so these are produced by the oracle
after it has been pinned (tests/test_oracle_pins.py).  Inputs are regenerated from seeds at test time; a fixture
stores the seed, a checksum of the regenerated inputs, and the expected outputs in float64-derived float32.
Nothing here imports or reads the reference.
"""
import hashlib
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import d2dmoe_oracle as O  # noqa: E402

CASES = {
    # name: shape of the layer; 'toy' is the shape the reference's own correctness print uses
    # (scripts/test_moe_implementations.py:39-55, 72-73)
    'toy': dict(B=5, T=2, D=64, E=4, Ed=32, W=128, act='relu', gated=False, taus=(0.5,), seed=101),
    'vit197': dict(B=1, T=197, D=768, E=128, Ed=24, W=128, act='relu', gated=False, taus=(0.1, 0.9), seed=102),
    'gpt64': dict(B=2, T=32, D=768, E=128, Ed=24, W=128, act='gelu', gated=False, taus=(0.9,), seed=103),
    'gated16': dict(B=1, T=16, D=256, E=16, Ed=64, W=32, act='gelu_tanh', gated=True, taus=(0.9,), seed=104),
}
KEEP_ROWS = 32


def make_inputs(case, dtype=torch.float32):
    c = CASES[case]
    p = O.make_layer_params(c['D'], c['E'], c['Ed'], c['W'], seed=c['seed'], gated=c['gated'],
                            bias=not c['gated'], dtype=torch.float32)
    g = torch.Generator().manual_seed(c['seed'] + 7)
    x = torch.randn(c['B'], c['T'], c['D'], generator=g)
    if 'last_bias' in p:
        p['last_bias'] = torch.randn(1, c['D'], generator=g) * 0.05
    if dtype != torch.float32:
        x = x.to(dtype)
        p = {k: v.to(dtype) for k, v in p.items()}
    return x, p


def inputs_checksum(x, p):
    h = hashlib.sha256()
    h.update(x.float().numpy().tobytes())
    for k in sorted(p):
        h.update(k.encode())
        h.update(p[k].float().numpy().tobytes())
    return h.hexdigest()


def main():
    for name, c in CASES.items():
        out = {}
        for dt_name, dt in (('f32', torch.float32), ('bf16', torch.bfloat16)):
            x, p = make_inputs(name, dt)
            out[f'checksum_{dt_name}'] = np.array(inputs_checksum(x, p))
            # norms in the storage dtype (what the gate sees), outputs from float64 math on the same stored values
            norms = O.router_forward(x, p['router_w1'], p['router_w2'])
            out[f'norms_{dt_name}'] = norms.float().numpy().reshape(-1, c['E'])[:KEEP_ROWS]
            for tau in c['taus']:
                routing = O.gate_dynk_max(norms, tau)
                o64 = O.layer_from_routing(x.double(), O.upcast(p), routing, c['act'], 'all')
                tag = f'{dt_name}_tau{tau}'
                r2 = routing.reshape(-1, c['E'])
                out[f'routing_bits_{tag}'] = np.packbits(r2.float().numpy().astype(np.uint8), axis=1)
                out[f'out_{tag}'] = o64.reshape(-1, c['D'])[:KEEP_ROWS].float().numpy()
                s, u, cnt = O.extract_indices(r2)
                off, tok = O.permutation_csr(r2)
                out[f'offsets_{tag}'] = off.numpy()
                out[f'token_idx_{tag}'] = tok.numpy()
                out[f'sort_crc_{tag}'] = np.array(hashlib.sha256(s.numpy().tobytes()).hexdigest())
                out[f'unsort_crc_{tag}'] = np.array(hashlib.sha256(u.numpy().tobytes()).hexdigest())
        path = os.path.join(HERE, f'{name}.npz')
        np.savez_compressed(path, **out)
        print(path, os.path.getsize(path), 'bytes')


if __name__ == '__main__':
    main()
