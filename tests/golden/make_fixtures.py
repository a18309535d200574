"""Writes the golden fixtures in this directory from the reference's own compiled CPU attention.

Run in a container that has the reference checkout:  make -C oracle ref && python tests/golden/make_fixtures.py
Every fixture stores its inputs and the outputs of oracle/_ref (the reference's Matrix / Softmax /
CausalSelfAttention sources compiled in place), so the tests need neither the reference nor this script.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib  # noqa: E402

# name: (q_heads, kv_heads, head_dim, seq_len, packs, col_start, pad_cols, seed, sigma_qk)
CASES = {
    "c1_tiny_fp32": (4, 4, 16, 48, 4, 0, 0, 0x5E17 + 1, 1.0),       # the quickstart LM attention shape
    "gqa_8q2kv_d8_T16": (8, 2, 8, 16, 1, 0, 0, 0x5E17 + 11, 1.0),    # shape of the reference's GQA host smoke
    "d64_T132": (2, 2, 64, 132, 1, 0, 0, 0x5E17 + 12, 1.0),          # ragged tail past two 64-wide tiles
    "gqa_d128_T96_B2": (2, 1, 128, 96, 2, 0, 0, 0x5E17 + 13, 1.0),   # head_dim 128, grouped K/V, two packs
    "d64_T256_B2_window": (1, 1, 64, 256, 2, 8, 24, 0x5E17 + 14, 1.0),  # pack window inside a wider matrix
    "d32_T80_sharp": (2, 2, 32, 80, 1, 0, 0, 0x5E17 + 15, 3.0),      # sigma 3 queries / keys: peaked softmax
}


def lcg_uniform(count, state):
    """The reference's smoke-test input recipe (Layers/CausalSelfAttention.cpp:566-574)."""
    out = np.empty(count, dtype=np.float32)
    for i in range(count):
        state = (state * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = np.float32(np.float32(state >> 8) / np.float32(16777216.0)) * np.float32(2.0) - np.float32(1.0)
    return out, state


def main():
    ref = oracle_lib.reference()
    if ref is None:
        raise SystemExit("oracle/_ref is not built (needs the reference checkout): make -C oracle ref")
    for name, (hq, hkv, d, t, packs, col0, pad, seed, sigma) in CASES.items():
        rng = np.random.default_rng(seed)
        stride = col0 + packs * t + pad
        q = (sigma * rng.standard_normal((hq * d, stride))).astype(np.float32)
        k = (sigma * rng.standard_normal((hkv * d, stride))).astype(np.float32)
        v = rng.standard_normal((hkv * d, stride)).astype(np.float32)
        g = rng.standard_normal((hq * d, stride)).astype(np.float32)
        res = oracle_lib.oracle_attention(q, k, v, g, q_heads=hq, kv_heads=hkv, head_dim=d, seq_len=t, pack_count=packs,
                                          col_start=col0, lib="ref")
        np.savez_compressed(os.path.join(HERE, name + ".npz"), q=q, k=k, v=v, d_out=g,
                            geometry=np.array([hq, hkv, d, t, packs, col0, stride], dtype=np.int64), **res)
        print(name, {key: val.shape for key, val in res.items()})

    # gemm / softmax known answers from the reference's Matrix::gemm and Softmax::applyInto
    rng = np.random.default_rng(0x5E17 + 20)
    kat = {}
    for tag, (m, kk, n, ta, tb) in {"nn_33x70x45": (33, 70, 45, False, False), "tn_96x16x96": (96, 16, 96, True, False),
                                    "nt_16x100x40": (16, 100, 40, False, True), "tt_37x41x29": (37, 41, 29, True, True)}.items():
        a = rng.standard_normal((kk, m) if ta else (m, kk)).astype(np.float32)
        b = rng.standard_normal((n, kk) if tb else (kk, n)).astype(np.float32)
        kat[f"gemm_{tag}_a"], kat[f"gemm_{tag}_b"] = a, b
        kat[f"gemm_{tag}_c"] = oracle_lib.gemm(a, b, ta, tb, lib="ref")
        kat[f"gemm_{tag}_flags"] = np.array([ta, tb], dtype=np.int64)
    logits = (4.0 * rng.standard_normal((50, 37))).astype(np.float32)
    logits[10:, 3] = -1e9
    kat["softmax_in"] = logits
    kat["softmax_out"] = oracle_lib.softmax_columns(logits, lib="ref")
    lcg, _ = lcg_uniform(64 * 16, 123)
    kat["lcg_seed123_first1024"] = lcg
    np.savez_compressed(os.path.join(HERE, "gemm_softmax_kat.npz"), **kat)
    print("gemm_softmax_kat", len(kat), "arrays")

    # RoPE tables and rotations from the reference's RotaryEmbedding (Layers/RotaryEmbedding.cpp)
    rng = np.random.default_rng(0x5E17 + 30)
    rope = {}
    for tag, (heads, d, t, base) in {"h3_d16_T40": (3, 16, 40, 10000.0), "h2_d64_T130": (2, 64, 130, 10000.0),
                                     "h1_d128_T33_base500k": (1, 128, 33, 500000.0)}.items():
        x = rng.standard_normal((heads * d, t)).astype(np.float32)
        cos, sin = oracle_lib.rope_tables(d, t + 7, base, lib="ref")
        rope[f"{tag}_geometry"] = np.array([heads, d, t, t + 7], dtype=np.int64)
        rope[f"{tag}_base"] = np.float32(base)
        rope[f"{tag}_x"], rope[f"{tag}_cos"], rope[f"{tag}_sin"] = x, cos, sin
        rope[f"{tag}_forward"] = oracle_lib.ref_rope_rotate(x, heads, d, t + 7, base)
        rope[f"{tag}_inverse"] = oracle_lib.ref_rope_rotate(x, heads, d, t + 7, base, inverse=True)
    np.savez_compressed(os.path.join(HERE, "rope_kat.npz"), **rope)
    print("rope_kat", sorted(rope))

    # the attention layer with real weights from the reference's CausalSelfAttention::forward / backward
    rng = np.random.default_rng(0x5E17 + 40)
    lay = {}
    for tag, (e, hq, hkv, d, t, base) in {"e64_h4_T48": (64, 4, 4, 16, 48, 10000.0), "e48_gqa6q2kv_d8_T33": (48, 6, 2, 8, 33, 10000.0),
                                          "e128_h2_d64_T70": (128, 2, 2, 64, 70, 500000.0)}.items():
        bound = 1.0 / np.sqrt(e)
        x = rng.standard_normal((e, t)).astype(np.float32)
        wq = rng.uniform(-bound, bound, (hq * d, e)).astype(np.float32)
        wk = rng.uniform(-bound, bound, (hkv * d, e)).astype(np.float32)
        wv = rng.uniform(-bound, bound, (hkv * d, e)).astype(np.float32)
        wo = rng.uniform(-bound, bound, (e, hq * d)).astype(np.float32)
        d_y = rng.standard_normal((e, t)).astype(np.float32)
        res = oracle_lib.layer(x, wq, wk, wv, wo, d_y, q_heads=hq, kv_heads=hkv, head_dim=d, rope_base=base,
                               rope_positions=t + 3, lib="ref")
        lay[f"{tag}_geometry"] = np.array([e, hq, hkv, d, t, t + 3], dtype=np.int64)
        lay[f"{tag}_base"] = np.float32(base)
        for key, val in dict(x=x, wq=wq, wk=wk, wv=wv, wo=wo, d_y=d_y, **res).items():
            lay[f"{tag}_{key}"] = val
    np.savez_compressed(os.path.join(HERE, "layer_kat.npz"), **lay)
    print("layer_kat", len(lay), "arrays")
    write_sparse_kat()


# name: (q_heads, kv_heads, head_dim, seq_len, packs, window, global_tokens)
SPARSE_CASES = {
    "smoke_h2_d16_T16_W4_G2": (2, 2, 16, 16, 1, 4, 2),    # runSparseComputeSmokeDemo(32, 2, 16, 32, 4, 2)
    "gqa_4q2kv_d8_T50_W7_G0": (4, 2, 8, 50, 1, 7, 0),      # window only, grouped heads
    "h1_d64_T140_W33_G5": (1, 1, 64, 140, 2, 33, 5),        # several 64-wide tiles, two packs
    "h2_d32_T70_W0_G9": (2, 2, 32, 70, 1, 0, 9),            # no window: the global tokens change nothing
    "h1_d128_T130_W1_G0": (1, 1, 128, 130, 1, 1, 0),        # window 1: every query sees only itself
    "h1_d16_T40_W100_G3": (1, 1, 16, 40, 1, 100, 3),        # window wider than the sequence
}


def write_sparse_kat():
    """Sliding-window / global-token masks from the reference's dense masked path (preferSparseCompute = false),
    plus the forward of its sparse-compute path, which differs only by summation order."""
    rng = np.random.default_rng(0x5E17 + 50)
    kat = {}
    for tag, (hq, hkv, d, t, packs, window, global_tokens) in SPARSE_CASES.items():
        stride = packs * t
        q = rng.standard_normal((hq * d, stride)).astype(np.float32)
        k = rng.standard_normal((hkv * d, stride)).astype(np.float32)
        v = rng.standard_normal((hkv * d, stride)).astype(np.float32)
        g = rng.standard_normal((hq * d, stride)).astype(np.float32)
        kw = dict(q_heads=hq, kv_heads=hkv, head_dim=d, seq_len=t, pack_count=packs, window=window,
                  global_tokens=global_tokens, lib="ref")
        # a window of 0 means "none" to the layer's constructor only through windowSize >= sequence length
        ref_kw = dict(kw, window=window if window > 0 else t)
        dense = oracle_lib.oracle_attention(q, k, v, g, prefer_sparse=False, **ref_kw)
        sparse = oracle_lib.oracle_attention(q, k, v, g, prefer_sparse=True, **ref_kw)
        kat[f"{tag}_geometry"] = np.array([hq, hkv, d, t, packs, window, global_tokens], dtype=np.int64)
        for key, val in dict(q=q, k=k, v=v, d_out=g).items():
            kat[f"{tag}_{key}"] = val
        for key, val in dense.items():
            kat[f"{tag}_dense_{key}"] = val
        for key, val in sparse.items():
            kat[f"{tag}_sparse_{key}"] = val
    np.savez_compressed(os.path.join(HERE, "sparse_kat.npz"), **kat)
    print("sparse_kat", len(kat), "arrays")


if __name__ == "__main__":
    if sys.argv[1:] == ["sparse"]:  # only the sparse-mask known answers
        if oracle_lib.reference() is None:
            raise SystemExit("oracle/_ref is not built (needs the reference checkout): make -C oracle ref")
        write_sparse_kat()
    else:
        main()
