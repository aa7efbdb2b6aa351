"""Writes the committed fixtures of tests/golden/.

    python tests/golden/make_fixtures.py

encoder_b2_l8_h2_e16_{relu,gelu}.npz: inputs, {0,1} masks and every named output
of the device-path graph, produced by stock torch ops + torch.autograd in fp64
(tests/torch_graph.py) -- not by the oracle, which these files pin.
philox_kat.npz: Random123 known-answer vectors for philox4x32_10 plus the first
64 16-bit fields for (seed=0x5EED, site=0..3, step=0), computed with the
pure-Python textbook Philox in this file.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from tests import torch_graph as tg  # noqa: E402


def philox_scalar(ctr, key):
    c = list(ctr); k = list(key)
    for _ in range(10):
        p0 = 0xD2511F53 * c[0]; p1 = 0xCD9E8D57 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & 0xffffffff, (p0 >> 32) ^ c[3] ^ k[1], p0 & 0xffffffff]
        k = [(k[0] + 0x9E3779B9) & 0xffffffff, (k[1] + 0xBB67AE85) & 0xffffffff]
    return c


def main():
    B, L, H, E = 2, 8, 2, 16
    for act in ('relu', 'gelu'):
        params, X, DY = tg.make_inputs(B, L, H, E, seed=2024, w_std=0.25, b_std=0.1)
        masks = tg.make_masks(B, L, H, E, 0.25, seed=2024)
        out = tg.run(params, X, DY, masks, act)
        blob = {'in_X': X.numpy(), 'in_DY': DY.numpy()}
        blob.update({'param_' + k: v.numpy() for k, v in params.items()})
        blob.update({'mask_' + k: v.numpy().astype(np.uint8) for k, v in masks.items()})
        blob.update({'out_' + k: v.numpy() for k, v in out.items()})
        np.savez_compressed(os.path.join(HERE, f'encoder_b2_l8_h2_e16_{act}.npz'), **blob)
    kat_in = np.array([[0, 0, 0, 0, 0, 0], [0xffffffff] * 6,
                       [0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344, 0xa4093822, 0x299f31d0]],
                      dtype=np.uint32)
    kat_out = np.array([[0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8],
                        [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd],
                        [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]], dtype=np.uint32)
    for i in range(3):
        assert philox_scalar(kat_in[i, :4].tolist(), kat_in[i, 4:].tolist()) == kat_out[i].tolist()
    seed = 0x5EED
    fields = np.zeros((4, 64), dtype=np.uint16)
    for site in range(4):
        for e in range(64):
            o = philox_scalar([e >> 3, 0, site, 0], [seed, 0])
            w = o[(e & 7) >> 1]
            fields[site, e] = (w >> 16) if (e & 1) else (w & 0xffff)
    np.savez_compressed(os.path.join(HERE, 'philox_kat.npz'), kat_in=kat_in, kat_out=kat_out,
                        seed=np.uint64(seed), fields=fields)


if __name__ == '__main__':
    main()
