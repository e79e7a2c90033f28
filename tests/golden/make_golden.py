"""Writes tests/golden/*.npz: small input/expected-output vectors for the three
data movements of the pcieThrough path.

The reference ships no golden data for this path (its tests fill the host pool
with a constant, pcieThrough/tests/test_transfer_kernel.py:32, or compare an
all-zero table with itself, pcieThrough/tests/test_gather.py:40), and its kernels
cannot run outside an Ascend NPU. The expected outputs here are therefore produced
by element-by-element Python loops written directly from the index formulas of

  pcieThrough/csrc/kernel/multi_layer_block_transfer_kernel.h:47,63-67
      layer[l][(h*T + t)*D + d] = host[((t*L + l)*H + h)*D + d]
  pcieThrough/csrc/kernel/gather.h:106-122
      dst[i, :] = table[ids[i], :]
  per plane: dst.index_copy_(0, dst_ids, src.index_select(0, src_ids))

using only numpy indexing of single elements; neither the C oracle nor torch is
involved, so the fixtures are an independent pin for both. Inputs are seeded
random bytes (every byte value, including NaN bit patterns of bf16/fp16/fp8).

Run:  python tests/golden/make_golden.py
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def transfer_case(seed, T, L, H, D, elem):
    rs = np.random.RandomState(seed)
    src = rs.randint(0, 256, size=T * L * H * D * elem).astype(np.uint8)
    out = np.zeros((L, H * T * D * elem), dtype=np.uint8)
    for t in range(T):
        for l in range(L):
            for h in range(H):
                for d in range(D):
                    for b in range(elem):
                        out[l, ((h * T + t) * D + d) * elem + b] = src[(((t * L + l) * H + h) * D + d) * elem + b]
    return dict(src=src, expected=out, geometry=np.array([T, L, H, D, elem], dtype=np.int64))


def table_transfer_case(seed, T, L, H, D, elem, packed_blocks, dev_blocks, n_pairs, to_packed):
    """Block-table form of the transfer, either direction, from single-element loops."""
    rs = np.random.RandomState(seed)
    packed = rs.randint(0, 256, size=(packed_blocks, T * L * H * D * elem)).astype(np.uint8)
    layers = rs.randint(0, 256, size=(L, dev_blocks, H * T * D * elem)).astype(np.uint8)
    pb = rs.permutation(packed_blocks)[:n_pairs]
    db = rs.permutation(dev_blocks)[:n_pairs]
    pairs = np.stack([pb, db], axis=1).astype(np.int64)
    packed_out, layers_out = packed.copy(), layers.copy()
    for j in range(n_pairs):
        for t in range(T):
            for l in range(L):
                for h in range(H):
                    for d in range(D * elem):
                        po = ((t * L + l) * H + h) * D * elem + d
                        lo = (h * T + t) * D * elem + d
                        if to_packed:
                            packed_out[int(pairs[j, 0]), po] = layers[l, int(pairs[j, 1]), lo]
                        else:
                            layers_out[l, int(pairs[j, 1]), lo] = packed[int(pairs[j, 0]), po]
    return dict(packed=packed, layers=layers, pairs=pairs, packed_expected=packed_out, layers_expected=layers_out,
                geometry=np.array([T, L, H, D, elem, int(to_packed)], dtype=np.int64))


def gather_case(seed, rows, row_bytes, n_ids, id_dtype):
    rs = np.random.RandomState(seed)
    table = rs.randint(0, 256, size=(rows, row_bytes)).astype(np.uint8)
    ids = rs.randint(0, rows, size=n_ids).astype(id_dtype)
    out = np.zeros((n_ids, row_bytes), dtype=np.uint8)
    for i in range(n_ids):
        for b in range(row_bytes):
            out[i, b] = table[int(ids[i]), b]
    return dict(table=table, ids=ids, expected=out)


def swap_case(seed, planes, src_blocks, dst_blocks, block_bytes, n_pairs):
    rs = np.random.RandomState(seed)
    src = rs.randint(0, 256, size=(planes, src_blocks, block_bytes)).astype(np.uint8)
    dst = rs.randint(0, 256, size=(planes, dst_blocks, block_bytes)).astype(np.uint8)
    s_ids = rs.permutation(src_blocks)[:n_pairs]
    d_ids = rs.permutation(dst_blocks)[:n_pairs]
    pairs = np.stack([s_ids, d_ids], axis=1).astype(np.int64)
    out = dst.copy()
    for p in range(planes):
        for j in range(n_pairs):
            for b in range(block_bytes):
                out[p, int(pairs[j, 1]), b] = src[p, int(pairs[j, 0]), b]
    return dict(src=src, dst_before=dst, pairs=pairs, expected=out)


def main():
    cases = {
        # (T, L, H, D, elem): tiny brute-force shapes covering element sizes 1, 2 and 4
        "transfer_T2_L3_H2_D16_e1": transfer_case(1, 2, 3, 2, 16, 1),
        "transfer_T2_L3_H2_D16_e2": transfer_case(2, 2, 3, 2, 16, 2),
        "transfer_T2_L3_H2_D16_e4": transfer_case(3, 2, 3, 2, 16, 4),
        "transfer_T5_L2_H3_D8_e2": transfer_case(4, 5, 2, 3, 8, 2),
        "transfer_T8_L4_H1_D128_e1": transfer_case(5, 8, 4, 1, 128, 1),
        "transfer_T3_L1_H1_D32_e2": transfer_case(6, 3, 1, 1, 32, 2),
        "transfer_T4_L2_H2_D7_e1": transfer_case(7, 4, 2, 2, 7, 1),
        "tabletransfer_in_T4_L3_H2_D16_e1": table_transfer_case(31, 4, 3, 2, 16, 1, 5, 4, 3, False),
        "tabletransfer_out_T4_L3_H2_D16_e1": table_transfer_case(32, 4, 3, 2, 16, 1, 5, 4, 3, True),
        "tabletransfer_in_T3_L2_H2_D32_e2": table_transfer_case(33, 3, 2, 2, 32, 2, 3, 6, 3, False),
        "tabletransfer_out_T3_L2_H2_D32_e2": table_transfer_case(34, 3, 2, 2, 32, 2, 3, 6, 3, True),
        "tabletransfer_out_T5_L2_H1_D6_e1": table_transfer_case(35, 5, 2, 1, 6, 1, 4, 4, 2, True),
        "gather_r37_b64_n19_i64": gather_case(11, 37, 64, 19, np.int64),
        "gather_r37_b64_n19_i32": gather_case(12, 37, 64, 19, np.int32),
        "gather_r9_b4096_n5_i64": gather_case(13, 9, 4096, 5, np.int64),
        "gather_r21_b1024_n40_i64": gather_case(14, 21, 1024, 40, np.int64),
        "gather_r13_b33_n7_i64": gather_case(15, 13, 33, 7, np.int64),
        "gather_r6_b8208_n4_i32": gather_case(16, 6, 8208, 4, np.int32),
        "swap_p3_s7_d9_b256_n5": swap_case(21, 3, 7, 9, 256, 5),
        "swap_p2_s5_d5_b4096_n5": swap_case(22, 2, 5, 5, 4096, 5),
        "swap_p2_s6_d4_b100_n3": swap_case(23, 2, 6, 4, 100, 3),
        "swap_p1_s4_d8_b8208_n4": swap_case(24, 1, 4, 8, 8208, 4),
    }
    for name, arrays in cases.items():
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
        print(name, {k: v.shape for k, v in arrays.items()})


if __name__ == "__main__":
    main()
