#!/usr/bin/env python3
"""Writes tests/golden/c5_matmul_checksum.json: checksums of the CPU oracle's result for BASELINE configuration 5
(int8 MatMul [4096,4096] x [4096,11008] with the per-column PPE and LeakyReLU, then Dequantize, then the fp16 Add),
computed once over the whole tensors.  The GPU test compares what the device produces with these values, so a run
does not have to trust the sampled rows alone.  Runs on the CPU only (about half a minute on 8 cores):

    python tests/golden/make_c5_checksum.py
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))


def digest(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    import oracle
    from vpux_plugin_amd import configs
    c = configs.c5_matmul()
    K = c["a"].shape[1]
    wt = oracle.make_weights_table(c["mult"], c["shift"], c["bias"], K)
    p = oracle.ppe(c["lrelu_mult"], c["lrelu_shift"], c["zp_out"], *c["clamp"])
    out = oracle.nce_matmul(c["a"], c["b_nk"], wt, p, zp_a=c["zp_a"])
    shipped = float(oracle.f16_to_f32(oracle.f32_to_f16(np.array([c["deq_scale"]], np.float32)))[0])
    deq = oracle.dequantize(out, shipped, c["deq_zp"])
    y = oracle.eltwise_f16("add", deq, c["residual"])
    rec = {
        "config": "c5_matmul seed 5, [4096,4096] x [11008,4096]^T, zp_a 3, LeakyReLU 1638/2^14, clamp [-128,127]",
        "matmul_i8": {"sha256": digest(out), "sum": int(out.astype(np.int64).sum()),
                      "row_sums_sha256": digest(out.astype(np.int64).sum(axis=1)),
                      "col_sums_sha256": digest(out.astype(np.int64).sum(axis=0))},
        "dequantize_f16_bits": {"sha256": digest(deq)},
        "add_f16_bits": {"sha256": digest(y)},
    }
    path = os.path.join(HERE, "c5_matmul_checksum.json")
    with open(path, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    print(json.dumps(rec, indent=1))


if __name__ == "__main__":
    main()
