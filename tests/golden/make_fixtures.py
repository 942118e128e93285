#!/usr/bin/env python3
"""Write tests/golden/*.npz from the COMPILED REFERENCE (oracle/_ref/liboilref*.so).

Run in the build container only (the reference tree is needed to build
oracle/_ref):   make -C oracle ref && python tests/golden/make_fixtures.py

Inputs follow the reference codec test's deterministic generator
(tests/test_block_codec.cpp:49-55, seeds 42 / 1337 / 1000+n, :176 tail sizes,
:247-250 the dense*0.85+0.6 transform) plus a x0.02 variant in the spirit of the
N(0,0.02) recipe; outputs are what the reference's quantize_block_all /
dequantize_block_all / oil4_gemm / oil8_gemm / gemv_*_tiled / quant_gemm
produced for them.  The fixtures hold data only: inputs, payload bytes and
output bit patterns.
"""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
TAILS = [1, 7, 15, 16, 17, 20, 21, 25, 26, 31, 32, 33, 39, 40, 63, 100, 128, 200, 255]

f32p = C.POINTER(C.c_float)
u8p = C.POINTER(C.c_uint8)
u16p = C.POINTER(C.c_uint16)


def p(a, t):
    return a.ctypes.data_as(t)


def codec_inputs():
    """(tag, weights) pairs."""
    cases = []
    w256 = O.xorshift_fill(256, 42) * np.float32(0.85) + np.float32(0.6)
    w512 = O.xorshift_fill(512, 1337) * np.float32(0.85) + np.float32(0.6)
    cases.append(("dense256", w256))
    cases.append(("dense512", w512))
    cases.append(("unit256", O.xorshift_fill(256, 99)))
    cases.append(("small256", O.xorshift_fill(256, 7) * np.float32(0.02)))
    cases.append(("zero256", np.zeros(256, dtype=np.float32)))
    spike = O.xorshift_fill(256, 11) * np.float32(0.02)
    spike[::37] *= np.float32(40.0)
    cases.append(("spiky256", spike))
    cases.append(("tiny256", O.xorshift_fill(256, 5) * np.float32(3e-8)))   # FP16 scale flushes
    for n in TAILS:
        cases.append((f"tail{n}", O.xorshift_fill(n, 1000 + n)))
        cases.append((f"tail{n}s", O.xorshift_fill(n, 2000 + n) * np.float32(0.02)))
    return cases


def make_codec():
    R = O.ref(True)
    assert R is not None, "build oracle/_ref first (make -C oracle ref)"
    rec = {k: [] for k in ("fmt", "n", "w_off", "idx_off", "idx_len", "cb_off", "cb_len", "dec_off")}
    tags, W, IDX, CB, DEC = [], [], [], [], []
    w_off = idx_off = cb_off = dec_off = 0
    for tag, w in codec_inputs():
        for fmt in range(15):
            idx, cb = O.ref_quantize_block(fmt, w)
            dec = O.ref_dequantize_block(fmt, idx, cb, w.size)
            tags.append(f"{tag}/{O.FORMAT_NAMES[fmt]}")
            rec["fmt"].append(fmt); rec["n"].append(w.size)
            rec["w_off"].append(w_off); rec["idx_off"].append(idx_off); rec["idx_len"].append(idx.size)
            rec["cb_off"].append(cb_off); rec["cb_len"].append(cb.size); rec["dec_off"].append(dec_off)
            IDX.append(idx); CB.append(cb); DEC.append(dec.view(np.uint32))
            idx_off += idx.size; cb_off += cb.size; dec_off += dec.size
        W.append(w.view(np.uint32)); w_off += w.size
    out = {k: np.asarray(v, dtype=np.int64) for k, v in rec.items()}
    out["tags"] = np.asarray(tags)
    out["w_bits"] = np.concatenate(W)
    out["idx"] = np.concatenate(IDX)
    out["cb"] = np.concatenate(CB)
    out["dec_bits"] = np.concatenate(DEC)
    # all 65536 half patterns through the reference's OIL16 decode
    hs = np.arange(65536, dtype=np.uint16)
    out["f16_to_f32_bits"] = O.ref_dequantize_block(5, hs.view(np.uint8), np.zeros(0, np.uint8), 65536).view(np.uint32)
    # float -> half: a spread of magnitudes, ties and specials through OIL16 encode
    rng = np.random.default_rng(20260803)
    f = np.concatenate([
        (rng.standard_normal(4096) * 10.0 ** rng.integers(-9, 6, 4096)).astype(np.float32),
        rng.integers(0, 1 << 32, 4096, dtype=np.uint64).astype(np.uint32).view(np.float32),
        ((np.arange(0, 4096, dtype=np.uint32) << 13) | 0x38000000 | 0x1000).view(np.float32),
        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 65504, 65520, 65519.99, 6.1e-5, 5.96e-8,
                  2.98e-8, 2.9e-8, 3.1e-8, 1e-10], dtype=np.float32)])
    h = np.concatenate([O.ref_quantize_block(5, f[s:s + 4096])[0] for s in range(0, f.size, 4096)])
    out["f32_in_bits"] = f.view(np.uint32)
    out["f32_to_f16"] = h.view(np.uint16)
    np.savez_compressed(os.path.join(HERE, "codec.npz"), **out)
    print("codec.npz:", len(tags), "cases")


def make_gemv():
    """Per format: a 32 x 768 matrix, reference payloads, reference decode,
    double-precision X.W^T of the reference-decoded weights (B = 3)."""
    R = O.ref(True)
    rows, cols, B = 32, 768, 3
    rng = np.random.default_rng(7)
    Wm = (rng.standard_normal(rows * cols) * 0.02).astype(np.float32)
    Wm[rng.integers(0, Wm.size, 200)] *= np.float32(8.0)
    X = rng.standard_normal((B, cols)).astype(np.float32)
    out = {"w_bits": Wm.view(np.uint32), "x_bits": X.view(np.uint32),
           "shape": np.array([rows, cols, B])}
    for fmt in range(15):
        idxs, cbs, decs = [], [], []
        for b in range(rows * cols // 256):
            idx, cb = O.ref_quantize_block(fmt, Wm[b * 256:(b + 1) * 256])
            idxs.append(idx); cbs.append(cb)
            decs.append(O.ref_dequantize_block(fmt, idx, cb, 256))
        Wd = np.concatenate(decs).reshape(rows, cols)
        Y = (X.astype(np.float64) @ Wd.astype(np.float64).T).astype(np.float32)
        name = O.FORMAT_NAMES[fmt]
        out[f"{name}/idx"] = np.concatenate(idxs)
        out[f"{name}/idx_len"] = np.array([a.size for a in idxs], dtype=np.int32)
        out[f"{name}/cb"] = np.concatenate(cbs) if sum(a.size for a in cbs) else np.zeros(0, np.uint8)
        out[f"{name}/cb_len"] = np.array([a.size for a in cbs], dtype=np.int32)
        out[f"{name}/y_bits"] = Y.view(np.uint32)
    np.savez_compressed(os.path.join(HERE, "block_gemv.npz"), **out)
    print("block_gemv.npz written")


def make_flat():
    R, RS = O.ref(True), O.ref(False)
    rng = np.random.default_rng(11)
    out = {}
    # oil8_gemm / oil4_gemm (AVX2 build)
    M, N, K = 3, 17, 300
    idx8 = rng.integers(0, 256, N * K, dtype=np.uint8).astype(np.uint8)
    cb8 = rng.standard_normal(256).astype(np.float32)
    act8 = rng.standard_normal(M * K).astype(np.float32)
    y8 = np.zeros(M * N, np.float32)
    R.ref_oil8_gemm(p(idx8, u8p), p(cb8, f32p), p(act8, f32p), p(y8, f32p), M, N, K)
    out.update({"oil8/idx": idx8, "oil8/cb_bits": cb8.view(np.uint32), "oil8/act_bits": act8.view(np.uint32),
                "oil8/y_bits": y8.view(np.uint32), "oil8/mnk": np.array([M, N, K])})
    pk = rng.integers(0, 256, M * N * K // 2 + 16, dtype=np.uint8).astype(np.uint8)
    cb16 = rng.standard_normal(16).astype(np.float16).view(np.uint16).copy()
    cb16[3] = 0x0001; cb16[5] = 0x83FF; cb16[9] = 0x0400
    act4 = rng.standard_normal(N * K).astype(np.float32)
    y4 = np.zeros(M * N, np.float32)
    R.ref_oil4_gemm(p(pk, u8p), p(cb16, u16p), p(act4, f32p), p(y4, f32p), M, N, K)
    out.update({"oil4/packed": pk, "oil4/cb16": cb16, "oil4/act_bits": act4.view(np.uint32),
                "oil4/y_bits": y4.view(np.uint32), "oil4/mnk": np.array([M, N, K])})
    # production GEMVs: scalar bodies (reference built without SIMD flags)
    Mg, Kg = 9, 301
    x = rng.standard_normal(Kg).astype(np.float32)
    ws = rng.integers(0, 256, Mg * ((Kg + 3) // 4), dtype=np.uint8).astype(np.uint8)
    w4 = rng.integers(0, 256, Mg * ((Kg + 1) // 2), dtype=np.uint8).astype(np.uint8)
    w8 = rng.integers(0, 256, Mg * Kg, dtype=np.uint8).astype(np.uint8)
    ys, yo4, yo8 = (np.zeros(Mg, np.float32) for _ in range(3))
    RS.ref_gemv_spark(p(ws, u8p), 0.37, p(x, f32p), p(ys, f32p), Mg, Kg)
    RS.ref_gemv_oil4(p(w4, u8p), p(cb16, u16p), 0.37, p(x, f32p), p(yo4, f32p), Mg, Kg)
    RS.ref_gemv_oil8(p(w8, u8p), p(cb8, f32p), 0.37, p(x, f32p), p(yo8, f32p), Mg, Kg)
    out.update({"prod/x_bits": x.view(np.uint32), "prod/mk": np.array([Mg, Kg]),
                "prod/w_spark": ws, "prod/w_oil4": w4, "prod/w_oil8": w8,
                "prod/y_spark_bits": ys.view(np.uint32), "prod/y_oil4_bits": yo4.view(np.uint32),
                "prod/y_oil8_bits": yo8.view(np.uint32)})
    # engines: default codebooks and quant_gemm
    Me, Ne, Ke = 3, 24, 40
    A = rng.standard_normal(Me * Ke).astype(np.float32)
    A[::7] = 0
    bq = rng.integers(0, 256, Ke * Ne, dtype=np.uint8).astype(np.uint8)
    out.update({"eng/A_bits": A.view(np.uint32), "eng/b": bq, "eng/mnk": np.array([Me, Ne, Ke])})
    for bits in (8, 4, 2):
        cb = np.zeros(256, np.float32)
        n = R.ref_engine_codebook(bits, p(cb, f32p))
        Cc = np.zeros(Me * Ne, np.float32)
        R.ref_engine_quant_gemm(bits, p(A, f32p), p(bq, u8p), p(Cc, f32p), Me, Ne, Ke)
        out[f"eng/cb{bits}_bits"] = cb[:n].view(np.uint32).copy()
        out[f"eng/c{bits}_bits"] = Cc.view(np.uint32)
    np.savez_compressed(os.path.join(HERE, "flat.npz"), **out)
    print("flat.npz written")


PLAN_TARGETS = [0.5, 1.0, 1.2, 1.5, 1.7, 1.925, 1.95, 2.0, 2.06, 2.075, 2.1, 2.2, 2.3, 2.5, 2.6, 2.75, 2.92, 3.0, 3.5,
                4.0, 4.12, 4.2, 4.3, 4.5, 5.0, 5.84, 6.0, 7.0, 7.675, 8.0, 8.24, 8.4, 8.5, 10, 12, 16, 20, 24, 32, 40]
PLAN_BLOCKS = [0, 1, 2, 3, 7, 10, 33, 100, 101, 257, 1000, 3906]


def plan_scores(kind, nb, rng):
    """Importance scores of a planner case: none, distinct, heavy ties, fewer scores than blocks."""
    if kind == 0:
        return np.zeros(0, np.float32)
    if kind == 1:
        return np.abs(rng.standard_normal(nb)).astype(np.float32)
    if kind == 2:
        return rng.integers(0, 4, nb).astype(np.float32)
    return np.abs(rng.standard_normal(max(nb // 2, 1))).astype(np.float32)


def mix_tensor(seed, n):
    """Weights whose blocks differ in scale and outliers, so that every tier of a mix gets used."""
    rng = np.random.default_rng(seed)
    w = rng.standard_normal(n).astype(np.float32) * np.float32(0.02)
    nb = (n + 255) // 256
    for b in range(nb):
        w[b * 256:(b + 1) * 256] *= np.float32(2.0 ** rng.integers(-3, 4))
        if rng.random() < 0.3:
            k = rng.integers(0, min(256, n - b * 256), 3)
            w[b * 256 + k] *= np.float32(25.0)
    return w


MIX_CASES = [("SPARK_MIX_Q0", 1, 64 * 256, 256, 0, 0), ("QUAD_SPARK_Q1", 2, 64 * 256, 256, 0, 0),
             ("SPARK_MIX_Q0", 3, 40 * 256 + 77, 256, 0, 0), ("QUAD_SPARK_Q1", 4, 96 * 100, 256, 96, 100),
             ("OIL8+OIL2_10_90", 5, 48 * 256, 256, 48, 256), ("QUAD_OIL2_OIL4_OIL8_OIL16", 6, 32 * 256, 256, 0, 0),
             ("SPARK_MIX_Q0", 7, 30 * 128, 128, 0, 0)]


def make_planner():
    """FormatPlanner::allocate / score_importance / FormatRegistry::allocate_mix_blocks and the
    registry tables, as the compiled reference (AVX2+FMA build) answers."""
    R = O.ref(True)
    assert R is not None, "build oracle/_ref first (make -C oracle ref)"
    R.ref_mix_allocate.restype = C.c_int64
    i64p, i32p = C.POINTER(C.c_int64), C.POINTER(C.c_int)
    out = {}
    # registry tables
    names, kinds, bpws, tiers, ratios, ntiers = [], [], [], [], [], []
    for kind in (0, 1, 2):
        i = 0
        while True:
            nm = C.create_string_buffer(64)
            bpw, nt = C.c_float(), C.c_int()
            t, r = np.zeros(4, np.uint8), np.zeros(4, np.float32)
            if not R.ref_registry_row(kind, i, nm, 64, C.byref(bpw), p(t, u8p), p(r, f32p), C.byref(nt)):
                break
            names.append(nm.value.decode()); kinds.append(kind); bpws.append(bpw.value)
            tiers.append(t); ratios.append(r); ntiers.append(nt.value)
            i += 1
    out["reg_name"] = np.array(names)
    out["reg_kind"] = np.array(kinds, np.int32)
    out["reg_bpw"] = np.array(bpws, np.float32)
    out["reg_tiers"] = np.stack(tiers)
    out["reg_ratios"] = np.stack(ratios)
    out["reg_ntiers"] = np.array(ntiers, np.int32)
    # planner cases: scores are regenerated from (seed, kind, nb) by the test
    rng = np.random.default_rng(5)
    meta, fm, ach, est = [], [], [], []
    for ti, target in enumerate(PLAN_TARGETS):
        for nb in PLAN_BLOCKS:
            for kind in range(4):
                s = plan_scores(kind, nb, rng)
                f = np.zeros(max(nb, 1), np.uint8)
                a, e, u = C.c_float(), C.c_float(), C.c_int()
                c7 = np.zeros(7, np.int32)
                R.ref_plan_allocate(C.c_float(target), p(s, f32p) if s.size else None, C.c_int64(s.size), C.c_int(nb),
                                    p(f, u8p), C.byref(a), C.byref(e), C.byref(u), p(c7, i32p))
                meta.append([ti, nb, kind, u.value] + list(c7))
                fm.append(f[:nb].copy()); ach.append(a.value); est.append(e.value)
    out["plan_meta"] = np.array(meta, np.int32)
    out["plan_fmts"] = np.concatenate(fm)
    out["plan_achieved"] = np.array(ach, np.float32)
    out["plan_estimated"] = np.array(est, np.float32)
    # importance scores
    rng = np.random.default_rng(6)
    sm, sw, sa, ss = [], [], [], []
    for n in (1, 255, 256, 257, 1000, 4096):
        for bs in (256, 64, 100):
            w = rng.standard_normal(n).astype(np.float32)
            a = rng.standard_normal(n).astype(np.float32)
            nb = (n + bs - 1) // bs
            for mode in (0, 1, 2):      # magnitude without activations, with activations, fisher
                sc = np.zeros(nb, np.float32)
                R.ref_score_importance(p(w, f32p), p(a, f32p) if mode else None, C.c_int64(n), C.c_int(bs),
                                       C.c_int(1 if mode == 2 else 0), p(sc, f32p))
                sm.append([n, bs, mode]); ss.append(sc)
            sw.append(w); sa.append(a)
    out["score_meta"] = np.array(sm, np.int32)
    out["score_w"] = np.concatenate(sw)
    out["score_a"] = np.concatenate(sa)
    out["score_out"] = np.concatenate(ss)
    # adaptive mix allocation (inputs regenerated by mix_tensor(seed, n) in the test)
    mm, mf, ms, ml = [], [], [], []
    for name, seed, n, bs, rows, cols in MIX_CASES:
        w = mix_tensor(seed, n)
        cap = n
        f, st, ln = np.zeros(cap, np.uint8), np.zeros(cap, np.int64), np.zeros(cap, np.int64)
        nb = R.ref_mix_allocate(name.encode(), p(w, f32p), C.c_int64(n), C.c_int(bs), C.c_int64(rows), C.c_int64(cols),
                                p(f, u8p), p(st, i64p), p(ln, i64p), C.c_int64(cap), None, None, None)
        assert nb > 0
        mm.append(nb); mf.append(f[:nb].copy()); ms.append(st[:nb].copy()); ml.append(ln[:nb].copy())
        print(name, "tiers used:", np.unique(f[:nb], return_counts=True))
    out["mix_nb"] = np.array(mm, np.int64)
    out["mix_fmts"] = np.concatenate(mf)
    out["mix_starts"] = np.concatenate(ms)
    out["mix_lens"] = np.concatenate(ml)
    np.savez_compressed(os.path.join(HERE, "planner.npz"), **out)
    print("planner.npz written")


CONTAINER_CONFIG = b'{"dim": 256, "note": "fixture"}'
CONTAINER_VERSION = (1 << 22) | (2 << 12) | 3
CONTAINER_FLAGS = 5


def container_tensors():
    """[(name, data, fmts, starts, lens)]: every wire format, a ragged tail, one-block-per-row blocks."""
    rng = np.random.default_rng(77)
    out = []
    w = (rng.standard_normal(32 * 256) * 0.3).astype(np.float32)
    out.append(("layers.0.attention.q_proj.weight", w, np.arange(32, dtype=np.uint8) % 15,
                np.arange(32, dtype=np.int64) * 256, np.full(32, 256, np.int64)))
    w = (rng.standard_normal(1000) * 0.05 + 1.0).astype(np.float32)
    out.append(("norm.weight", w, np.array([6, 5, 11, 4], np.uint8), np.arange(4, dtype=np.int64) * 256,
                np.array([256, 256, 256, 232], np.int64)))
    w = (rng.standard_normal(64 * 100) * 0.1).astype(np.float32)
    out.append(("tok_embeddings.weight", w, (np.arange(64, dtype=np.uint8) * 7) % 15,
                np.arange(64, dtype=np.int64) * 100, np.full(64, 100, np.int64)))
    return out


def make_container():
    """tests/golden/mixed.oil written by the reference's OILWriter, and what its OILReader reads back."""
    R = O.ref(True)
    assert R is not None, "build oracle/_ref first (make -C oracle ref)"
    R.ref_oil_read_tensor.restype = C.c_int64
    i64p = C.POINTER(C.c_int64)
    ts = container_tensors()
    names = (C.c_char_p * len(ts))(*[t[0].encode() for t in ts])
    counts = np.array([len(t[2]) for t in ts], np.uint32)
    data = np.concatenate([t[1] for t in ts])
    fmts = np.concatenate([t[2] for t in ts])
    base = np.cumsum([0] + [t[1].size for t in ts])[:-1]
    starts = np.concatenate([t[3] + b for t, b in zip(ts, base)])
    lens = np.concatenate([t[4] for t in ts])
    path = os.path.join(HERE, "mixed.oil")
    cfg = np.frombuffer(CONTAINER_CONFIG, np.uint8)
    rc = R.ref_oil_write(path.encode(), C.c_uint32(CONTAINER_VERSION), C.c_uint32(CONTAINER_FLAGS), p(cfg, u8p),
                         C.c_uint32(cfg.size), C.c_uint32(len(ts)), names, counts.ctypes.data_as(C.POINTER(C.c_uint32)),
                         p(data, f32p), p(fmts, u8p), p(starts, i64p), p(lens, i64p), C.c_uint32(fmts.size))
    assert rc == 0, rc
    out = {}
    for k, t in enumerate(ts):
        dec = np.zeros(t[1].size, np.float32)
        n = R.ref_oil_read_tensor(path.encode(), t[0].encode(), p(dec, f32p), C.c_int64(dec.size))
        assert n == dec.size, (t[0], n)
        out[f"decoded{k}"] = dec.view(np.uint32)
    nb, nt, st, cnt = C.c_uint32(), C.c_uint32(), C.c_uint32(), C.c_uint32()
    assert R.ref_oil_meta(path.encode(), ts[2][0].encode(), C.byref(nb), C.byref(nt), C.byref(st), C.byref(cnt)) == 0
    out["meta"] = np.array([nb.value, nt.value, st.value, cnt.value], np.int64)
    np.savez_compressed(os.path.join(HERE, "container.npz"), **out)
    print("mixed.oil", os.path.getsize(path), "bytes; container.npz written", out["meta"])


MOE_ROUTE_CASES = [(64, 8, 2), (5, 4, 1), (33, 16, 4), (7, 3, 3), (100, 8, 8), (16, 64, 6)]
MOE_SHAPE = dict(T=10, E=3, K=2, D=256, F=512)


def moe_route_logits(T, E, kind, rng):
    lg = rng.standard_normal((T, E)).astype(np.float32)
    if kind == 1:
        lg = np.round(lg)                       # many exact ties
    if kind == 2:
        lg[:] = np.float32(0.5)                 # all experts equal
    return lg


def moe_experts(seed, E, D, F, fmts=(3, 3, 3)):
    """Per expert: (payload, blocks) of gate [F][D], up [F][D], down [D][F], quantized with the oracle's
    quantizer (byte-identical to the reference's), and their decoded matrices."""
    rng = np.random.default_rng(seed)
    packs, dense = [], []
    for e in range(E):
        pe, de = [], []
        for (r, c), f in zip(((F, D), (F, D), (D, F)), fmts):
            w = (rng.standard_normal(r * c) * (1.0 / np.sqrt(c))).astype(np.float32)
            payload, blocks = O.quantize_tensor(w, f)
            pe.append((payload, blocks))
            de.append(O.dequant_blocks(payload, blocks).reshape(r, c))
        packs.append(pe)
        dense.append(de)
    return packs, dense


def make_moe():
    """softmax_with_topk and moe_dispatch_batched as the compiled reference answers."""
    R = O.ref_moe()
    assert R is not None, "build oracle/_ref first (make -C oracle ref)"
    out = {}
    rng = np.random.default_rng(1)
    pr, ix, wt = [], [], []
    for T, E, k in MOE_ROUTE_CASES:
        for kind in range(3):
            lg = moe_route_logits(T, E, kind, rng)
            p_, i_, w_ = O.softmax_topk(lg, k, fn=R.ref_softmax_topk)
            pr.append(p_.view(np.uint32).ravel()); ix.append(i_.ravel()); wt.append(w_.view(np.uint32).ravel())
    out["route_probs"] = np.concatenate(pr)
    out["route_idx"] = np.concatenate(ix)
    out["route_w"] = np.concatenate(wt)
    sh = MOE_SHAPE
    _, dense = moe_experts(11, sh["E"], sh["D"], sh["F"])
    rng = np.random.default_rng(12)
    x = rng.standard_normal((sh["T"], sh["D"])).astype(np.float32)
    lg = rng.standard_normal((sh["T"], sh["E"])).astype(np.float32)
    _, idx, w = O.softmax_topk(lg, sh["K"], fn=R.ref_softmax_topk)
    w[2, 0] = 0.0            # a dropped pair
    idx[4, 1] = -1           # an entry outside the expert range
    idx[6, 1] = idx[6, 0]    # the same expert twice
    o, z, dr = O.moe_dispatch(x, [d[0] for d in dense], [d[1] for d in dense], [d[2] for d in dense], idx, w,
                              fn=R.ref_moe_dispatch)
    out["disp_x"] = x
    out["disp_idx"] = idx
    out["disp_w"] = w
    out["disp_out"] = o.view(np.uint32)
    out["disp_z"] = np.array([z], np.float32)
    out["disp_dropped"] = np.array([dr], np.int64)
    np.savez_compressed(os.path.join(HERE, "moe.npz"), **out)
    print("moe.npz written; dropped", dr, "z", z)


ENGINE_DENSE = dict(M=3, N=96, K=80, block=128)


def engine_dense_inputs(kind):
    """(A, B, scales) for Oil1 / Spark / OIL16 / OIL32 engine quant_gemm cases; some activations are zero."""
    sh = ENGINE_DENSE
    rng = np.random.default_rng(40 + kind)
    A = rng.standard_normal((sh["M"], sh["K"])).astype(np.float32)
    A[:, ::7] = 0.0
    flat = sh["K"] * sh["N"]
    scales = None
    if kind == 1:
        B = rng.standard_normal((flat + 31) // 32).astype(np.float32)
    elif kind == 32:
        B = rng.standard_normal(flat).astype(np.float32)
    elif kind == 16:
        B = rng.standard_normal(flat).astype(np.float16).view(np.uint16).copy()
        B[:8] = [0x8000, 0x0000, 0x0001, 0x83FF, 0x7C00, 0xFC00, 0x0400, 0x3C00]     # signed zero, subnormals, infinities
        A[:, 0] = 0.0                                                                # keep the infinities out of the sums
        B[4 * sh["N"]: 4 * sh["N"] + 0] = 0
        B[4:6] = [0x3800, 0xB800]
    else:
        B = rng.integers(0, 256, (flat + 3) // 4).astype(np.uint8)
        scales = np.abs(rng.standard_normal((flat + sh["block"] - 1) // sh["block"])).astype(np.float32)
    return A, B, scales


def engine_dequant_inputs(bits):
    n = {8: 1001, 4: 999, 2: 1003}[bits]
    rng = np.random.default_rng(60 + bits)
    return rng.integers(0, 256, (n * bits + 7) // 8).astype(np.uint8), n


def engine_block_inputs(bits):
    n, block = 777, 64
    rng = np.random.default_rng(70 + bits)
    idx = rng.integers(0, 1 << bits, n).astype(np.uint8)
    nb = (n + block - 1) // block
    scales = rng.standard_normal(nb * (2 if bits == 4 else 1)).astype(np.float32)
    return idx, scales, n, block


def make_engines():
    R = O.ref(True)
    assert R is not None, "build oracle/_ref first (make -C oracle ref)"
    sh = ENGINE_DENSE
    out = {}
    for kind in (1, 3, 16, 32):
        A, B, scales = engine_dense_inputs(kind)
        Cc = O.engine_dense_gemm(kind, A, B, sh["M"], sh["N"], sh["K"], scales, sh["block"], fn=R.ref_engine_dense_gemm)
        out[f"c{kind}"] = Cc.view(np.uint32)
    # dequant_tensor (packed codes) and dequantize_per_block (one index byte per weight), default codebooks
    for bits in (8, 4, 2):
        cb = np.zeros(256, np.float32)
        ncb = R.ref_engine_codebook(bits, p(cb, f32p))
        out[f"cb{bits}"] = cb[:ncb].view(np.uint32)
        idx, n = engine_dequant_inputs(bits)
        o = np.zeros(n, np.float32)
        R.ref_engine_dequant(C.c_int(bits), p(idx, u8p), C.c_int64(n), None, C.c_int64(0), p(o, f32p))
        out[f"dq{bits}"] = o.view(np.uint32)
    for bits in (8, 4):
        idx, scales, n, block = engine_block_inputs(bits)
        o = np.zeros(n, np.float32)
        R.ref_engine_dequant(C.c_int(bits), p(idx, u8p), C.c_int64(n), p(scales, f32p), C.c_int64(block), p(o, f32p))
        out[f"pb{bits}"] = o.view(np.uint32)
    np.savez_compressed(os.path.join(HERE, "engines.npz"), **out)
    print("engines.npz written")



KV_CASES = [  # max_seq, heads, dim, block, appends (tokens per call); even and odd tokens, tokens shorter than a block
    (64, 2, 32, 64, [5, 1, 1, 3]), (24, 8, 128, 64, [7, 1, 1]), (32, 1, 48, 64, [3, 2, 1, 1]), (32, 1, 16, 32, [1, 1, 1, 4]),
    (40, 3, 11, 64, [4, 1, 2]), (16, 2, 64, 128, [16]), (16, 1, 24, 77, [2, 2, 2]), (20, 5, 7, 32, [3, 1, 1, 1, 5]),
    (8, 1, 64, 64, [1] * 8), (8, 2, 64, 32, [4, 4])]
KV_BLOCK_SIZES = [1, 2, 3, 7, 16, 31, 32, 33, 64, 100, 127, 128, 200, 5000]


def kv_inputs(i):
    ms, h, d, block, lens = KV_CASES[i]
    rng = np.random.default_rng(900 + i)
    tot = sum(lens)
    k = rng.standard_normal((tot, h * d)).astype(np.float32)
    v = (rng.standard_normal((tot, h * d)) * 3).astype(np.float32)
    if i % 3 == 1:
        k[:, : h * d // 2] = 0.25          # constant chunks
    return k, v


def kv_block_inputs(j):
    n = KV_BLOCK_SIZES[j % len(KV_BLOCK_SIZES)]
    rng = np.random.default_rng(950 + j)
    x = rng.standard_normal(n).astype(np.float32)
    kind = j % 6
    if kind == 1: x *= 1e-6
    if kind == 2: x = (np.round(x * 2) / 2).astype(np.float32)
    if kind == 3: x[:] = x[0]
    if kind == 4: x *= 1e4
    if kind == 5: x = (x * 1e-3).astype(np.float32); x[::3] = 0
    return x


def make_kv():
    R = O.ref(True)
    assert R is not None, "build oracle/_ref first (make -C oracle ref)"
    R.ref_kv_float_to_half.restype = C.c_uint16
    R.ref_kv_float_to_half.argtypes = [C.c_float]
    # through dequantize_block_oil4 so that the floats come back through memory, signalling NaNs intact
    h2f = np.zeros((4096, 16), np.float32)
    codes = np.arange(16, dtype=np.uint8)
    for b in range(4096):
        cb = np.arange(b * 16, b * 16 + 16, dtype=np.uint16)
        R.ref_kv_dequantize_block(C.c_void_p(codes.ctypes.data), C.c_void_p(cb.ctypes.data), C.c_void_p(h2f[b].ctypes.data), C.c_int64(16))
    out = {"h2f": h2f.ravel().view(np.uint32)}
    fbits = kv_f2h_inputs()
    out["f2h"] = np.array([R.ref_kv_float_to_half(float(f)) for f in fbits.view(np.float32)], np.uint16)
    for j in range(84):
        cb, codes = O.kv_quantize_block(kv_block_inputs(j), fn=R.ref_kv_quantize_block)
        out[f"qcb{j}"], out[f"qcodes{j}"] = cb, codes
    for i, (ms, h, d, block, lens) in enumerate(KV_CASES):
        k, v = kv_inputs(i)
        tot = sum(lens)
        for r, (st, en) in enumerate([(0, tot), (1, tot - 1), (0, tot + 5)]):
            ko, vo, sb, cl = O.ref_kv_run(ms, h, d, block, k, v, lens, st, en)
            out[f"k{i}_{r}"], out[f"v{i}_{r}"] = ko.view(np.uint32), vo.view(np.uint32)
            out[f"meta{i}_{r}"] = np.array([sb, cl], np.int64)
    np.savez_compressed(os.path.join(HERE, "kv.npz"), **out)
    print("kv.npz written")


def kv_f2h_inputs():
    rng = np.random.default_rng(970)
    bits = np.concatenate([rng.integers(0, 2 ** 32, 20000, dtype=np.uint64).astype(np.uint32),
                           np.arange(0x33000000, 0x33000000 + 1000, dtype=np.uint32),
                           np.arange(0x38000000, 0x38000000 + 20000, 7, dtype=np.uint32),
                           np.array([0, 0x80000000, 0x7f800000, 0xff800000, 0x477fe000, 0x477ff000, 0x47800000, 0x38800000,
                                     0x387fffff, 0x33800000, 0x337fffff], dtype=np.uint32)])
    f = bits.view(np.float32)
    return bits[~np.isnan(f)]


# ---------------------------------------------------------------- SPARK lookup kernels
# (kind, M, N, K): the shape of the reference's own test (tests/test_protected.cpp:177-192), odd K for TL1's tail,
# K that is not a multiple of 12 for TL2's last group, a long row, one output
TL_CASES = [(1, 4, 4, 16), (1, 3, 5, 33), (1, 2, 3, 7), (1, 5, 2, 255), (1, 1, 1, 1), (1, 2, 2, 1200), (1, 6, 9, 4096),
            (2, 4, 4, 36), (2, 3, 5, 33), (2, 2, 3, 9), (2, 5, 2, 255), (2, 1, 1, 3), (2, 2, 2, 1200), (2, 6, 9, 4095)]


def tl_inputs(i):
    kind, M, N, K = TL_CASES[i]
    rng = np.random.default_rng(5100 + i)
    w = rng.integers(0, 256, size=M * N * O.tl_row_bytes(kind, K), dtype=np.uint8)
    a = (rng.standard_normal((N, K)) * rng.choice([1e-3, 1.0, 50.0], size=(N, 1))).astype(np.float32)
    a[0, :] = np.where(rng.random(K) < 0.5, -1.0, 1.0) * np.abs(a[0, :]).max()   # a saturated row: TL1's pair sums clamp
    if N > 1:
        a[1, :] = 0.0                                                            # all-zero row: the 1e-10 floor
    return w, a


def make_tl():
    R = O.ref()
    out = {"cases": np.array(TL_CASES, dtype=np.int32)}
    for i, (kind, M, N, K) in enumerate(TL_CASES):
        w, a = tl_inputs(i)
        out[f"w{i}"], out[f"a{i}"] = w, a
        out[f"out{i}"] = O.tl_gemm(kind, w, a, M, N, K, fn=R.ref_tl_gemm).view(np.uint32)
    np.savez_compressed(os.path.join(HERE, "tl.npz"), **out)
    print("tl.npz written")


if __name__ == "__main__":
    which = sys.argv[1:] or ["codec", "gemv", "flat", "planner", "container", "moe", "engines", "kv", "tl"]
    for name in which:
        {"codec": make_codec, "gemv": make_gemv, "flat": make_flat, "planner": make_planner,
         "container": make_container, "moe": make_moe, "engines": make_engines, "kv": make_kv, "tl": make_tl}[name]()
