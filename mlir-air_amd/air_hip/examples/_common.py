import numpy as np

from .. import bf16


def draw_l1_weights(rows, k, gs):
    """The examples' draw order after np.random.seed(...): nibbles, scales, zero points
    (matvec_int4_packed.py:345-350)."""
    q_unp = np.random.randint(0, 16, size=(rows, k), dtype=np.uint8)
    a_q = (q_unp[:, 0::2] | (q_unp[:, 1::2] << 4)).astype(np.uint8)
    n_groups = k // gs
    a_s = bf16.from_f32(np.random.uniform(0.005, 0.02, size=(n_groups, rows)))
    a_z = np.random.randint(7, 9, size=(n_groups, rows), dtype=np.uint8)
    return a_q, a_s, a_z
