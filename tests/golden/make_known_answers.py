#!/usr/bin/env python3
"""Writes tests/golden/known_answers.json: small known-answer vectors for every
operator of the path, each worked out BY HAND from the reference's source text
(file:line cited per case) -- none is produced by running the reference, the
oracle or the kernels.  The reference's own tests hold no golden data for this
path (their inputs are unseeded random tensors), so these are the fixtures.

    python tests/golden/make_known_answers.py
"""
import json
import os

HALF = 0.5   # noise 0.5 makes `(x - mn) * scale + noise - 0.5` deterministic: round-half-even of (x - mn) * scale

CASES = [
    # ---- Philox4x32-10: Random123's published kat_vectors -------------------------------------
    {"op": "philox", "ctr": [0, 0, 0, 0], "key": [0, 0],
     "out": [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]},
    {"op": "philox", "ctr": [0xFFFFFFFF] * 4, "key": [0xFFFFFFFF] * 2,
     "out": [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]},
    {"op": "philox", "ctr": [0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], "key": [0xA4093822, 0x299F31D0],
     "out": [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]},

    # ---- pack with given min / scale (quantization_cuda_kernel.cu:63-94, length :107-113) ------
    # 2 bits, 4 rows of one column share a byte: 0 | 1<<2 | 2<<4 | 3<<6 = 0xE4; + 1 pad byte
    {"op": "pack", "bits": 2, "x": [[0], [1], [2], [3]], "mn": [0, 0, 0, 0], "scale": [1, 1, 1, 1],
     "noise": [[HALF]] * 4, "packed": [0xE4, 0x00]},
    # 1 bit, 8 rows x 2 columns: column 0 has rows 0,2,4,6 set (0x55), column 1 rows 1,3,5,7 (0xAA)
    {"op": "pack", "bits": 1, "x": [[1, 0], [0, 1]] * 4, "mn": [0] * 8, "scale": [1] * 8,
     "noise": [[HALF, HALF]] * 8, "packed": [0x55, 0xAA, 0x00]},
    # ragged: 5 rows at 2 bits -> N_round = 8, second byte holds row 4 alone in bits 0-1
    {"op": "pack", "bits": 2, "x": [[0], [1], [2], [3], [2]], "mn": [0] * 5, "scale": [1] * 5,
     "noise": [[HALF]] * 5, "packed": [0xE4, 0x02, 0x00]},
    # 4 bits, 3 rows x 2 columns: rows 0,1 pair up (low nibble = row 0), row 2 stands alone
    {"op": "pack", "bits": 4, "x": [[0, 15], [7, 8], [3, 12]], "mn": [0] * 3, "scale": [1] * 3,
     "noise": [[HALF, HALF]] * 3, "packed": [0x70, 0x8F, 0x03, 0x0C, 0x00]},
    # 8 bits: one byte per element; 127.5 rounds half-to-even to 128 (__float2int_rn, :89)
    {"op": "pack", "bits": 8, "x": [[0, 127.5, 255], [1, 2, 3]], "mn": [0, 0], "scale": [1, 1],
     "noise": [[HALF] * 3] * 2, "packed": [0, 128, 255, 1, 2, 3, 0]},
    # the noise decides: 0.25 + 0.74 - 0.5 = 0.49 -> 0, 0.25 + 0.76 - 0.5 = 0.51 -> 1
    {"op": "pack", "bits": 8, "x": [[0.25], [0.25]], "mn": [0, 0], "scale": [1, 1],
     "noise": [[0.74], [0.76]], "packed": [0, 1, 0]},
    # min and scale are applied per row: (x - 10) * 0.5
    {"op": "pack", "bits": 2, "x": [[10, 12, 14, 16]], "mn": [10], "scale": [0.5],
     "noise": [[HALF] * 4], "packed": [0, 1, 2, 3, 0]},

    # ---- row statistics + scale + pack in one call (ops.py:39, 61-83) ---------------------------
    # mn 0, mx 3: scale = fl(1/3) * 3 = 1.0 in fp32 (torch evaluates int / tensor as reciprocal * int)
    {"op": "minmax_pack", "bits": 2, "x": [[0, 1, 2, 3]], "noise": [[HALF] * 4],
     "packed": [0, 1, 2, 3, 0], "scale_bf16": [0x3F80], "min_bf16": [0x0000]},
    # constant row: mx - mn = 0 -> scale inf, (x - mn) * inf = NaN, fmax(NaN, 0) = 0 -> all codes 0
    {"op": "minmax_pack", "bits": 2, "x": [[5] * 8], "noise": [[HALF] * 8],
     "packed": [0] * 9, "scale_bf16": [0x7F80], "min_bf16": [0x40A0]},
    # negative minimum: mn -2, mx 6, scale = fl(1/8) * 15 = 1.875; codes rne([0, 3.75, 7.5, 15]) = [0, 4, 8, 15]
    {"op": "minmax_pack", "bits": 4, "x": [[-2, 0, 2, 6]], "noise": [[HALF] * 4],
     "packed": [0, 4, 8, 15, 0], "scale_bf16": [0x3FF0], "min_bf16": [0xC000]},

    # ---- unpack (quantization_cuda_kernel.cu:158-185): code / scale + min ------------------------
    {"op": "unpack", "bits": 2, "packed": [0xE4, 0x00], "scale": [2, 2, 2, 2], "mn": [-1, -1, -1, -1],
     "N": 4, "G": 1, "out": [[-1.0], [-0.5], [0.0], [0.5]]},
    {"op": "unpack", "bits": 1, "packed": [0x55, 0xAA, 0x00], "scale": [0.25] * 8, "mn": [1] * 8,
     "N": 8, "G": 2, "out": [[5, 1], [1, 5]] * 4},
    {"op": "unpack", "bits": 4, "packed": [0x70, 0x8F, 0x03, 0x0C, 0x00], "scale": [1, 2, 4], "mn": [0, 0, 10],
     "N": 3, "G": 2, "out": [[0, 15], [3.5, 4], [10.75, 13]]},
    {"op": "unpack", "bits": 8, "packed": [0, 128, 255, 1, 2, 3, 0], "scale": [255, 1], "mn": [0, -1],
     "N": 2, "G": 3, "out": [[0, 0.501960813999176, 1], [0, 1, 2]]},   # 128/255 in fp32

    # ---- ReLU / LeakyReLU with a 1-bit mask (quantization_cuda_kernel.cu:237-331, 339-435) ------
    # bit i of the mask word = (x[i] > 0); -0.0 and 0 are not > 0
    {"op": "relu", "x": [-1, 2, 0, 3, -0.0, 0.5], "y": [0, 2, 0, 3, 0, 0.5], "mask": [0x2A],
     "dy": [1, 2, 3, 4, 5, 6], "dx": [0, 2, 0, 4, 0, 6]},
    {"op": "leaky_relu", "slope": 0.25, "x": [-4, 2], "y": [-1, 2], "mask": [0x2], "dy": [8, 8], "dx": [2, 8]},

    # ---- dropout (quantization_cuda_kernel.cu:442-594): keep = u > p, y = x * keep / (1 - p) ------
    {"op": "dropout", "p": 0.5, "x": [1, 2, 3, 4], "noise": [0.5, 0.51, 0.1, 0.9], "y": [0, 4, 0, 8], "mask": [0xA],
     "dy": [1, 1, 1, 1], "dx": [0, 2, 0, 2]},
    # p = 0.25: pinv = fl(1 / 0.75) = 1.33333337; 3 * pinv = 4.00000012 -> fp32 4.0; backward 3 / 0.75 = 4
    {"op": "dropout", "p": 0.25, "x": [3, 3], "noise": [0.3, 0.2], "y": [4, 0], "mask": [0x1],
     "dy": [3, 3], "dx": [4, 0]},

    # ---- ReLU -> dropout -> minmax_pack as one call (the chain of the three above) ----------------
    # relu: [0,2,3,0,5,6,7,8]; element 2 dropped: y = [0,4,0,0,10,12,14,16]; joint mask bits 1,4,5,6,7 = 0xF2;
    # mn 0, mx 16: scale = fl(1/16) * 3 = 0.1875; codes rne([0,.75,0,0,1.875,2.25,2.625,3]) = [0,1,0,0,2,2,3,3]
    {"op": "relu_dropout_pack", "p": 0.5, "bits": 2, "x": [[-1, 2, 3, -4, 5, 6, 7, 8]],
     "act_noise": [[0.9, 0.9, 0.1, 0.9, 0.9, 0.9, 0.9, 0.9]], "noise": [[HALF] * 8],
     "y": [[0, 4, 0, 0, 10, 12, 14, 16]], "mask": [0xF2], "packed": [0, 1, 0, 0, 2, 2, 3, 3, 0],
     "scale_bf16": [0x3E40], "min_bf16": [0x0000]},

    # ---- batch norm -> ReLU -> dropout -> minmax_pack as one call (layers.py:340-369 ahead of the chain) ----
    # per column (x - mean) * mult + shift, all exact in fp32:
    #   row 0 -> [-1, 2, 3, -4, 5, 6, 7, 8], the case above; row 1 -> [0.5, 0, 1, 0, 0, 6, 16, 0], nothing dropped:
    #   y = [1, 0, 2, 0, 0, 12, 32, 0], mask bits 8, 10, 13, 14; mn 0, mx 32: scale = fl(1/32) * 3 = 0.09375;
    #   codes rne([.09375, 0, .1875, 0, 0, 1.125, 3, 0]) = [0, 0, 0, 0, 0, 1, 3, 0]; byte d = row 0 | row 1 << 2
    {"op": "bn_relu_dropout_pack", "p": 0.5, "bits": 2,
     "x": [[0.25, 2, 3, 4, 1, 10, 0, 0], [1, 0, -1, 2, 0, 10, 9, -8]],
     "mean": [1, 0, -1, 2, 0, 10, 0, -8], "mult": [2, 1, 0.5, -2, 5, 1, 1, 1], "shift": [0.5, 0, 1, 0, 0, 6, 7, 0],
     "act_noise": [[0.9, 0.9, 0.1, 0.9, 0.9, 0.9, 0.9, 0.9], [0.9] * 8], "noise": [[HALF] * 8] * 2,
     "y": [[0, 4, 0, 0, 10, 12, 14, 16], [1, 0, 2, 0, 0, 12, 32, 0]], "mask": [0x65F2],
     "packed": [0, 1, 0, 0, 2, 6, 15, 3, 0], "scale_bf16": [0x3E40, 0x3DC0], "min_bf16": [0x0000, 0x0000]},

    # ---- CSR SpMM (spmm_cuda.cu:27-104, reducer.cuh:43-85) -----------------------------------------
    # A = [[1,0,2],[0,0,0],[0,3,0]]; row 1 is empty -> 0 (mean divides by max(count, 1))
    {"op": "spmm", "reduce": "sum", "rowptr": [0, 2, 2, 3], "col": [0, 2, 1], "val": [1, 2, 3],
     "X": [[1, 2], [3, 4], [5, 6]], "out": [[11, 14], [0, 0], [9, 12]]},
    {"op": "spmm", "reduce": "mean", "rowptr": [0, 2, 2, 3], "col": [0, 2, 1], "val": [1, 2, 3],
     "X": [[1, 2], [3, 4], [5, 6]], "out": [[5.5, 7], [0, 0], [9, 12]]},
    {"op": "spmm", "reduce": "sum", "rowptr": [0, 2, 2, 3], "col": [0, 2, 1], "val": None,
     "X": [[1, 2], [3, 4], [5, 6]], "out": [[6, 8], [0, 0], [3, 4]]},
    # max: row 0 compares 1*[1,2] with 2*[5,6]; the arg is the entry index, nnz (= 3) for the empty row
    {"op": "spmm", "reduce": "max", "rowptr": [0, 2, 2, 3], "col": [0, 2, 1], "val": [1, 2, 3],
     "X": [[1, 2], [3, 4], [5, 6]], "out": [[10, 12], [0, 0], [9, 12]], "arg": [[1, 1], [3, 3], [2, 2]]},
    {"op": "spmm", "reduce": "min", "rowptr": [0, 2, 2, 3], "col": [0, 2, 1], "val": [1, 2, 3],
     "X": [[1, 2], [3, 4], [5, 6]], "out": [[1, 2], [0, 0], [9, 12]], "arg": [[0, 0], [3, 3], [2, 2]]},
    # edge-value gradient (spmm_cuda.cu:172-209): out[e] = X[col[e]] . grad[row[e]]  (/ row length for mean)
    {"op": "sddmm", "reduce": "sum", "rowptr": [0, 2, 2, 3], "col": [0, 2, 1], "X": [[1, 2], [3, 4], [5, 6]],
     "grad": [[1, 1], [0, 0], [2, 0]], "out": [3, 11, 6]},
    {"op": "sddmm", "reduce": "mean", "rowptr": [0, 2, 2, 3], "col": [0, 2, 1], "X": [[1, 2], [3, 4], [5, 6]],
     "grad": [[1, 1], [0, 0], [2, 0]], "out": [1.5, 5.5, 6]},

    # ---- random projection (ops.py:107-125): X R and X_r R^T ---------------------------------------
    {"op": "rp", "X": [[1, 2, 3], [4, 5, 6]], "R": [[1, 0], [0, -1], [1, 1]],
     "fwd": [[4, 1], [10, 1]], "bwd_of_fwd": [[4, -1, 5], [10, -1, 11]]},
    # projection then quantisation in one call (ops.py:141-149), 2 bits, noise 0.5, on the product above:
    # row 0: mn 1, mx 4, scale = fl(1/3) * 3 = 1.0, codes [3, 0]; row 1: mn 1, mx 10, scale = fl(fl(1/9) * 3) =
    # 0.33333334 (0x3EAAAAAB, bf16 0x3EAB), codes rne([3.0000002, 0]) = [3, 0]; byte d = row 0 | row 1 << 2
    {"op": "rp_pack", "bits": 2, "X": [[1, 2, 3], [4, 5, 6]], "R": [[1, 0], [0, -1], [1, 1]], "noise": [[HALF] * 2] * 2,
     "packed": [15, 0, 0], "scale_bf16": [0x3F80, 0x3EAB], "min_bf16": [0x3F80, 0x3F80]},
]

if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "known_answers.json")
    with open(path, "w") as f:
        json.dump(CASES, f, indent=1)
    print(f"wrote {len(CASES)} cases to {path}")
