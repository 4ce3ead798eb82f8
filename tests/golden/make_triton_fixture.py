"""Turns the output of tests/triton_promotion_probe.py (run on a GPU box: ``python tests/triton_promotion_probe.py
probe.npz cuda``) into the compact fixture tests/golden/triton_scale_chain_probe.npz:

    python tests/golden/make_triton_fixture.py probe.npz

Kept: the scale-chain results for zero and every bf16 value with 2^-8 <= |x| < 2^8 (as bf16 bit patterns), and
every seventh of the 65536 near-threshold stage-2 cases.  The fp16 half of the probe goes to
tests/golden/triton_scale_chain_probe_fp16.npz the same way (fp16 bit patterns, the same range of |x|)."""
import os
import sys

import numpy as np


def bf16_bits(a):
    return (np.ascontiguousarray(a, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)


def main(src):
    r = np.load(src)
    x = r["x"]
    keep = np.nonzero(((np.abs(x) >= 2.0 ** -8) & (np.abs(x) < 2.0 ** 8)) | (x == 0))[0]
    out = {"x_bf16_bits": bf16_bits(x[keep])}
    for name in ("d128", "d64", "odd"):
        out[f"sm_{name}"] = r[f"sm_{name}"]
        for kind in ("constexpr", "runtime"):
            a = r[f"{kind}_{name}"][keep]
            assert np.array_equal(a, (bf16_bits(a).astype(np.uint32) << 16).view(np.float32))  # bf16-valued
            out[f"{kind}_{name}_bf16_bits"] = bf16_bits(a)
    sl = slice(0, None, 7)  # 7 is coprime with the 16 offsets per anchor: every offset stays represented
    out.update(s2_dot=r["s2_dot"][sl], s2_anchor_bf16_bits=bf16_bits(r["s2_anchor"][sl]), s2_qk_bf16_bits=bf16_bits(r["s2_qk"][sl]),
               s2_hit=r["s2_hit"][sl], s2_sm=r["s2_sm"], s2_theta=r["s2_theta"])
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "triton_scale_chain_probe.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes")
    if "h_x" not in r:
        return
    f16_bits = lambda a: np.ascontiguousarray(a, dtype=np.float32).astype(np.float16).view(np.uint16)
    x = r["h_x"]
    keep = np.nonzero(((np.abs(x) >= 2.0 ** -8) & (np.abs(x) < 2.0 ** 8)) | (x == 0))[0][::4]  # every fourth value
    out = {"x_f16_bits": f16_bits(x[keep])}
    for name in ("d128", "d64", "odd"):
        out[f"sm_{name}"] = r[f"sm_{name}"]
        for kind in ("constexpr", "runtime"):
            a = r[f"h_{kind}_{name}"][keep]
            assert np.array_equal(a, f16_bits(a).view(np.float16).astype(np.float32))  # fp16-valued
            out[f"{kind}_{name}_f16_bits"] = f16_bits(a)
    out.update(s2_dot=r["h_s2_dot"][sl], s2_anchor_f16_bits=f16_bits(r["h_s2_anchor"][sl]), s2_qk_f16_bits=f16_bits(r["h_s2_qk"][sl]),
               s2_hit=r["h_s2_hit"][sl], s2_sm=r["s2_sm"], s2_theta=r["s2_theta"])
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "triton_scale_chain_probe_fp16.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main(sys.argv[1])
