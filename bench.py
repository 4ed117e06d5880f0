#!/usr/bin/env python3
"""Benchmark of the CKKS polynomial hot path on one MI355X.

Headline workload (the batched RNS NTT configuration): 32 polynomials x 24
limbs of 50-bit primes at N = 2^16, uint64 coefficients uniform mod q_i from a
seeded generator, already resident in HBM; one step = forward NTT of the whole
batch followed by the inverse NTT (a round trip).  `value` is algorithmic
GB/s: 16 bytes per coefficient per transform (one read + one write of every
limb) x 2 transforms / step time.

The same line also reports, as extra fields, HMult+relinearise+rescale pairs/s
(L=24, k=7 special primes, dnum=3) and hoisted rotations/s, the per-kernel
roofline of the dominant NTT kernel measured with HIP events on the library's
stream, and the CPU oracle timed on this host for the same workload.

Prints exactly one JSON line on stdout.
"""
import argparse
import json
import os
import subprocess
import tempfile
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ace-compiler_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
# HBM bytes per launch of each NTT kernel on this workload, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this script, calibrated against the plain copy of the same buffer
# (profiles/ntt_batch_N65536_L24.md).  Algorithmic bytes per launch are 805306368.
TRAFFIC_BYTES = {'ntt_fwd_strided': 805524267, 'ntt_fwd_chunk_run': 818408808, 'ntt_inv_half_run': 853094267, 'ntt_inv_strided': 805770728}
N, LIMBS, POLYS = 65536, 24, 32
CFG = (N, LIMBS, 50, 50, 3)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def settle(g, fn, ms=60.0):
    """Untimed calls of fn until the GPU has been busy for `ms` milliseconds: the part's clocks (and with them every
    kernel time) settle only after some tens of milliseconds of load, and a measurement that starts on an idle GPU
    reads up to 10 % slow."""
    g.sync()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(4):
            fn()
        g.sync()


def time_region(g, fn, reps):
    """Average milliseconds per call of fn over reps calls, by HIP events on the library's stream, after the
    clocks have settled under the same load."""
    settle(g, fn)
    g.timer_start()
    for _ in range(reps):
        fn()
    return g.timer_stop_ms() / reps


def cpu_baseline(x_host, idx, budget_s):
    """The NTT round trip on the host, one thread, on a bounded sample of the same batch: the reference's own
    Ftt_fwd / Ftt_inv where the compiled reference (oracle/_ref/ref_driver) is present, else the oracle's port."""
    import refdrv

    per_poly = LIMBS * N
    if refdrv.available():
        s = refdrv.RefSession(*CFG)
        k = s.add(refdrv.OP_TIME_NTT, LIMBS, int(budget_s * 1000), 0, 0, idx, x_host[:per_poly])
        _, res = s.run()
        trips, ns = int(res[k][0]), int(res[k][1])
        assert (res[k][2:] == x_host[:per_poly]).all()
        gbs = trips * per_poly * 16 * 2 / (ns * 1e-9) / 1e9
        return {"value": round(gbs, 4), "unit": "GB/s", "cores": 1, "kind": "reference",
                "sample": "%d round trips of one polynomial of the batch (%d limbs) through the reference's Ftt_fwd / "
                          "Ftt_inv, %.1f s, single thread, gcc -O3" % (trips, LIMBS, ns * 1e-9)}
    from oracle_lib import Oracle

    o = Oracle(*CFG)
    done, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < budget_s:  # walk the batch, again from the start if time is left
        p = done % POLYS
        s = slice(p * per_poly, (p + 1) * per_poly)
        y = o.ntt(x_host[s], idx)
        z = o.intt(y, idx)
        assert (z == x_host[s]).all()
        done += 1
    dt = time.perf_counter() - t0
    o.close()
    gbs = done * per_poly * 16 * 2 / dt / 1e9
    return {"value": round(gbs, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "%d polynomial round trips (x%d limbs each) drawn from the same %d-polynomial batch, "
                      "%.1f s, single thread, gcc -O3" % (done, LIMBS, POLYS, dt)}


def keyswitch_leg(g, o, swk_host, cts_host, swk, cts):
    """16 independent HMult + relinearise + rescale at l=24, k=7, dnum=3, one batched call; after the timed region
    one pair of the batch is compared with the oracle."""
    import headline

    extra = {}
    level = g.L
    pairs = headline.PAIRS
    log("key-switch leg: %d ciphertext pairs, one relinearisation key" % pairs)
    stride = level * N
    ops = headline.hmult_operands(g, cts, level, pairs, stride)
    ostride = (level - 1) * N
    r0, r1 = g.alloc(pairs * ostride), g.alloc(pairs * ostride)

    def hmult_batch():
        g.mul_relin_rescale_batch(r0, r1, ostride, ops[0], ops[1], ops[2], ops[3], stride, swk, level, pairs)

    hmult_batch()
    ms = time_region(g, hmult_batch, 5)
    extra["keyswitch_ops_per_s"] = round(pairs / (ms * 1e-3), 1)
    extra["hmult_relin_rescale_ms"] = round(ms / pairs, 4)
    # compulsory traffic per op: 96 input + 46 output limbs of 512 KiB (the key's 186 limbs are shared by the batch)
    extra["keyswitch_hbm_frac"] = round((142 * pairs + 186) * N * 8 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
    p = 11  # one pair of the timed batch against the oracle
    t0 = time.perf_counter()
    w0, w1 = o.mul_relin_rescale(*(headline.shifted_host(c, p, g.primes[:level]) for c in cts_host), swk_host, level)
    extra["keyswitch_cpu_oracle_s_per_op"] = round(time.perf_counter() - t0, 3)
    ok = bool((r0.view(p * ostride, ostride).get() == w0).all() and (r1.view(p * ostride, ostride).get() == w1).all())
    extra["keyswitch_verified"] = ok
    assert ok, "HMult+relinearise+rescale of pair %d differs from the oracle" % p

    def hmult_single():
        g.mul_relin_rescale(r0, r1, cts[0], cts[1], cts[2], cts[3], swk, level)

    hmult_single()
    extra["hmult_relin_rescale_single_ms"] = round(time_region(g, hmult_single, 10), 4)
    for b in ops + [r0, r1]:
        b.free()
    return extra


def rotation_leg(g, o, swk_host, cts_host, swk, cts):
    """32 rotations of one ciphertext with the raised digits of c1 shared (hoisting), one batched call; after the
    timed region one rotation of the batch is compared with the oracle."""
    import headline

    extra = {}
    level = g.L
    nrot = headline.ROTATIONS
    log("rotation leg: %d rotations of one ciphertext, hoisted ModUp" % nrot)
    rots = headline.rotation_indices()
    keys = headline.rotation_keys(g, swk, nrot)
    ks = [g.find_automorphism_index(r) for r in rots]
    orders = [g.automorphism_order(k, True) for k in ks]
    n = level * N
    s0, s1 = g.alloc(nrot * n), g.alloc(nrot * n)
    f = lambda: g.rotate_batch(s0, s1, cts[0], cts[1], keys, orders, level)
    f()
    ms = time_region(g, f, 5)
    extra["rotations_per_s"] = round(nrot / (ms * 1e-3), 1)
    extra["rotate_batch_ms"] = round(ms, 3)
    # compulsory traffic: 186 key limbs in + 48 result limbs out per rotation, 48 input limbs once
    extra["rotation_hbm_frac"] = round((234 * nrot + 48) * N * 8 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
    i = 21  # one rotation of the timed batch against the oracle
    t0 = time.perf_counter()
    digits = o.precomp(cts_host[1], level, True)
    t1 = time.perf_counter()
    w0, w1 = o.fast_rotate(cts_host[0], digits, headline.rotation_key_host(g, swk_host, i),
                           o.automorphism_order(ks[i], True), level)
    extra["rotation_cpu_oracle_s"] = {"hoisted_modup": round(t1 - t0, 3), "per_rotation": round(time.perf_counter() - t1, 3)}
    ok = bool((s0.view(i * n, n).get() == w0).all() and (s1.view(i * n, n).get() == w1).all())
    extra["rotation_verified"] = ok
    assert ok, "rotation %d of the batch differs from the oracle" % i
    for b in keys + orders + [s0, s1]:
        b.free()
    return extra


def bootstrap_leg():
    """One CKKS bootstrap on the host runtime (tests/programs/bootstrap_program, a separate process): N=65536,
    34 limbs (q0 60 bits, scale 56 bits: the parameters of the reference's published ResNet-20 run, whose 19
    bootstraps take 784.03 s on one CPU thread), fully packed, refreshed to level 15 as that program asks."""
    exe = os.path.join(ROOT, "tests", "programs", "bootstrap_program")
    if not os.path.exists(exe):
        return {"bootstrap": {"error": "tests/programs/bootstrap_program is not built"}}
    try:
        r = subprocess.run([exe, "65536", "33", "60", "56", "192", "32768", "15", "1"], capture_output=True, text=True,
                           timeout=240)
        f = r.stdout.split()
        vals = dict(zip(f[0::2], f[1::2]))
        ms = float(vals["ms"])
        # the margin against 1e-3 over the keys and messages (there is no bit-level counterpart to compare with):
        # four more seeds, the last of them with a census of the bootstrap's calls for the CPU estimate
        errs = [float(vals["max_err"])]
        census = os.path.join(tempfile.mkdtemp(prefix="ace_census_"), "census.txt")
        for seed in (2, 3, 4, 5):
            rs = subprocess.run([exe, "65536", "33", "60", "56", "192", "32768", "15", str(seed)], capture_output=True,
                                text=True, timeout=240, env=dict(os.environ, ACE_HIP_CENSUS=census) if seed == 5 else None)
            fs = rs.stdout.split()
            errs.append(float(fs[fs.index("max_err") + 1]))
        est = reference_cpu_estimate(census + ".bootstrap", (65536, 34, 60, 56, 3))
        return {"bootstrap": {"workload": "one bootstrap, N=65536, 34 limbs (60/56 bits), 32768 slots, to level 15",
                              "ms": ms, "first_call_ms": float(vals["first_ms"]),
                              "max_err": float(vals["max_err"]), "max_err_over_5_seeds": max(errs),
                              "cpu_estimate": est, "exit_status": r.returncode,
                              "published_cpu_ms": round(784.03e3 / 19, 1),
                              "published_cpu_note": "the reference's published run, same chain, one CPU thread of "
                                                    "other hardware: not a same-run baseline"}}
    except Exception as e:  # the headline line must still be printed
        return {"bootstrap": {"error": repr(e)[:200]}}


def resnet20_leg():
    """The reference's generated ResNet-20/CIFAR-10 program (rtlib/ant/dataset/resnet20_cifar10_pre.onnx.inc,
    N=65536, 34 limbs, 197 rotation keys, 19 bootstraps), built unchanged against the host runtime where the reference
    tree was present, on the 60/56-bit chain the reference's build script compiles it with
    (scripts/build_resnet20_cifar10.sh:13-14,32; the committed program carries the compiler's defaults 51/46, on which
    its bootstraps are far outside their precision).  Its weight file is not available, so the weights are
    pseudo-random (RT_HIP_SYNTHETIC_WEIGHTS): the run measures time per image, and a second run under other keys
    measures how far the logits depend on the keys and the noise."""
    exe = os.path.join(ROOT, "oracle", "_ref", "models", "resnet20_cifar10_pre.onnx")
    if not os.path.exists(exe):
        return {"resnet20": {"skipped": "the model binary is built only where the reference tree is present"}}
    try:
        env = dict(os.environ, RT_HIP_SYNTHETIC_WEIGHTS="0.33", MODEL_Q0_BITS="60", MODEL_SF_BITS="56", MODEL_KEY_SEED="11")
        # three images one after another: the first pays for encoding every weight plaintext, the later ones find
        # the encoded polynomials in HBM
        r = subprocess.run([exe, "3", "32", "32", "10", "1", "3"], capture_output=True, text=True, timeout=400, env=env)
        line = [l for l in r.stdout.splitlines() if l.startswith("context_s")][0].split()
        vals = dict(zip(line[0::2], (float(v) for v in line[1::2])))
        later = [float(l.split()[5]) for l in r.stdout.splitlines() if l.startswith("image ")]
        logits = [float(v) for v in [l for l in r.stdout.splitlines() if l.startswith("output:")][0].split()[1:]]
        out = {"workload": "ResNet-20 CIFAR-10 inference, the reference's generated program on the 60/56-bit chain, "
                           "synthetic weights and images, three images one after another",
               "main_graph_s": vals["main_graph_s"],
               "main_graph_s_note": "first image: every weight plaintext is encoded on the fly, as the reference does "
                                    "for every image (the like-for-like figure)",
               "keygen_s": vals["keygen_s"], "input_s": vals["input_s"], "output_s": vals["output_s"],
               "exit_status": r.returncode, "published_cpu_s": 1453.96,
               "published_cpu_note": "the reference's published run: same chain, trained weights, one CPU thread of "
                                     "other hardware; not a same-run baseline"}
        if later:
            out["main_graph_s_later_images"] = later
            out["later_images_note"] = "later images reuse the encoded weight plaintexts kept in HBM"
        # Images on three host threads of one process, as the reference's driver runs a batch (`#pragma omp
        # parallel for`, dataset/resnet_cifar.main.inc:81-112): a later image's launches are too small for the
        # machine, launches of independent images overlap.  One set of keys, tables and kept plaintexts; a context of
        # the family (stream, scratch, buffers) per thread.  The first image runs alone, nine more three at a time.
        rt = subprocess.run([exe, "3", "32", "32", "10", "1", "10"], capture_output=True, text=True, timeout=400,
                            env=dict(env, MODEL_THREADS="3"))
        line = [l for l in rt.stdout.splitlines() if l.startswith("threads ")]
        if rt.returncode == 0 and line:
            w = line[0].split()
            out["three_threads"] = {"threads": int(w[1].rstrip(":")), "images": int(w[2]), "wall_s": float(w[5]),
                                    "s_per_image": float(w[7]),
                                    "note": "images 2-10 on three host threads of one process sharing one set of keys "
                                            "(30 GB) and the kept weight plaintexts; wall time of the batch / images"}
        # what the same calls would cost in the reference's C code on this host (an estimate: see the function)
        census = os.path.join(tempfile.mkdtemp(prefix="ace_census_"), "census.txt")
        rc = subprocess.run([exe, "3", "32", "32", "10", "1"], capture_output=True, text=True, timeout=400,
                            env=dict(env, ACE_HIP_CENSUS=census, RT_HIP_PLAINTEXT_CACHE_GB="0"))
        est = reference_cpu_estimate(census, (65536, 34, 60, 56, 3)) if rc.returncode == 0 else None
        if est:
            out["cpu_estimate"] = est
        env["MODEL_KEY_SEED"] = "22"
        r2 = subprocess.run([exe, "3", "32", "32", "10", "1"], capture_output=True, text=True, timeout=400, env=env)
        again = [float(v) for v in [l for l in r2.stdout.splitlines() if l.startswith("output:")][0].split()[1:]]
        out["logits_first_image"] = logits
        out["logit_spread_under_other_keys"] = max(abs(x - y) for x, y in zip(logits, again))
        # the same generated program over the plain-float stand-in runtime, on the host: what the logits must be
        shadow = exe + "_shadow"
        if os.path.exists(shadow):
            rs = subprocess.run([shadow, "3", "32", "32", "10", "1"], capture_output=True, text=True, timeout=200, env=env)
            if rs.returncode == 0:
                want = [float(v) for v in [l for l in rs.stdout.splitlines() if l.startswith("output:")][0].split()[1:]]
                out["logits_plain_float_run"] = want
                out["max_difference_from_plain_float_run"] = round(max(abs(x - y) for x, y in zip(logits, want)), 6)
        return {"resnet20": out}
    except Exception as e:
        return {"resnet20": {"error": repr(e)[:200]}}


def reference_cpu_estimate(census_path, chain, seconds_cap=40.0):
    """What a program's calls would take in the reference's own C code on this host, one thread: the counts of a
    census of the library's entry points (ACE_HIP_CENSUS: entry point, level, second size, calls) times the
    reference functions each entry point stands for, those timed by the compiled reference (oracle/_ref/ref_driver:
    Hw_modadd / Hw_modmul / Hw_modmuladd / Hw_modmul_scalar / Hw_rotate / Ftt_fwd / Ftt_inv per limb, Decomp_modup,
    Mod_down, Rescale, Dot_prod, Encode_at_level_with_sf) at nine levels of the same chain and interpolated between
    them.  An estimate, labelled so: the reference's CKKS layer cannot be built here, so its bootstrap and ciphertext
    operations enter as the sums of the polynomial functions they are made of (evaluator.c, bootstrap.c)."""
    import numpy as np
    import refdrv

    if not refdrv.available() or not os.path.exists(census_path):
        return None
    N, L, q0, sf, parts = chain
    s = refdrv.RefSession(*chain)
    levels = sorted({3, 6, 10, 14, 18, 22, 26, 30, L} & set(range(3, L + 1)))
    ks = [s.add(refdrv.OP_TIME_PRIMITIVES, lv, 7) for lv in levels]
    info, res = s.run()
    K, part_size = info["K"], info["part_size"]
    tab = np.array([[float(v) * 1e-9 for v in res[k]] for k in ks])  # [level sample][primitive] seconds
    names = ["add", "mul", "mac", "mul_scalar", "rot", "ntt", "intt", "decomp_modup", "mod_down", "rescale", "dot", "encode"]
    per_limb = {n: float(np.median(tab[:, i])) for i, n in enumerate(names[:7])}

    def t(name, level):
        return float(np.interp(level, levels, tab[:, names.index(name)]))

    nd = lambda lv: -(-lv // part_size)
    a_, m_, c_, ms_, r_ = (per_limb[k] for k in ("add", "mul", "mac", "mul_scalar", "rot"))
    switch = lambda lv: 2 * t("dot", lv) + 2 * t("mod_down", lv)
    precomp = lambda lv: nd(lv) * t("decomp_modup", lv)
    cost = {
        "hw_add": lambda lv, b: a_, "hw_mul": lambda lv, b: m_, "hw_mac": lambda lv, b: c_,
        "hw_add_scalar": lambda lv, b: a_, "hw_mul_scalar": lambda lv, b: ms_, "hw_mac_scalar": lambda lv, b: ms_ + a_,
        "ace_hw_rotate": lambda lv, b: r_,
        "ace_zero": lambda words, b: words * 8 / 5e9, "ace_copy": lambda words, b: words * 16 / 5e9,
        "ace_encode": lambda lv, b: max(b, 1) * t("encode", lv),
        "ace_mod_down": lambda lv, b: max(b, 1) * t("mod_down", lv),
        "ace_rescale": lambda lv, b: t("rescale", lv),
        "ace_decomp_modup": lambda lv, b: t("decomp_modup", lv), "ace_mod_up": lambda lv, b: t("decomp_modup", lv),
        "ace_precomp": lambda lv, b: max(b, 1) * precomp(lv),
        "poly_add": lambda limbs, b: limbs * a_, "poly_mul": lambda limbs, b: limbs * m_,
        "poly_add_scalars": lambda lv, b: lv * a_, "poly_mul_scalars": lambda lv, b: lv * ms_,
        "ace_ext_rotate": lambda lv, b: 2 * t("dot", lv) + (lv + K) * (2 * r_ + a_),
        "ace_ext_plain_mac": lambda lv, b: b * 2 * (lv + K) * (m_ + a_),
        "ace_ciph_wsum": lambda lv, b: b * 2 * lv * (ms_ + a_),
        "ace_mul_ciph3": lambda lv, b: lv * (4 * m_ + a_),
        "ace_relin": lambda lv, b: precomp(lv) + switch(lv) + 2 * lv * a_,
        "ace_rescale_ciph": lambda lv, b: 2 * t("rescale", lv),
        "ace_mul_relin_rescale": lambda lv, b: max(b, 1) * (lv * (4 * m_ + a_) + precomp(lv) + switch(lv) + 2 * lv * a_ + 2 * t("rescale", lv)),
        "ace_mul_relin_double_rescale": lambda lv, b: lv * (4 * m_ + a_) + precomp(lv) + switch(lv) + 4 * lv * a_ + 2 * t("rescale", lv),
        "ace_mul_relin_double_add_rescale": lambda lv, b: lv * (4 * m_ + a_) + precomp(lv) + switch(lv) + 5 * lv * a_ + 2 * t("rescale", lv),
        "ace_mod_down_pair_rescale": lambda lv, b: 2 * t("mod_down", lv) + 2 * t("rescale", lv),
        "ace_rotate_batch": lambda lv, b: precomp(lv) + b * (switch(lv) + lv * (a_ + 2 * r_)),
        "ace_fast_rotate": lambda lv, b: switch(lv) + lv * (a_ + 2 * r_),
        "ace_fast_switch_key": lambda lv, b: switch(lv), "ace_dot_prod": lambda lv, b: t("dot", lv),
        "ace_extend": lambda lv, b: lv * ms_,
        "ace_ntt": lambda limbs, b: limbs * per_limb["ntt"], "ace_intt": lambda limbs, b: limbs * per_limb["intt"],
        "ace_transform_from_level0": lambda lv, b: lv * a_,
        "ace_mod_down_rescale": lambda lv, b: t("mod_down", lv) + t("rescale", lv),
        "ace_reduce_rescale_modup": lambda lv, b: t("mod_down", lv) + t("rescale", lv) + t("decomp_modup", lv),
        "ace_poly_automorphism": lambda limbs, b: limbs * r_,
    }
    total, by_entry, unknown = 0.0, {}, set()
    for line in open(census_path):
        name, a, b, n = line.split()
        f = cost.get(name)
        if not f:
            unknown.add(name)
            continue
        sec = int(n) * f(int(a), int(b))
        total += sec
        by_entry[name] = by_entry.get(name, 0.0) + sec
    top = dict(sorted(((k, round(v, 1)) for k, v in by_entry.items()), key=lambda kv: -kv[1])[:8])
    return {"cpu_estimate_s": round(total, 1), "cores": 1, "kind": "estimate from the reference's own functions",
            "largest_parts_s": top, "not_counted": sorted(unknown),
            "method": "calls of one image by entry point and level (ACE_HIP_CENSUS, weight plaintexts encoded every "
                      "time as the reference does) x the reference's Hw_* / Ftt / Decomp_modup / Mod_down / Rescale / "
                      "Dot_prod / Encode timed on this host at %d levels of the chain, gcc -O3, one thread" % len(levels)}


def keyswitch_cpu_reference(level):
    """The reference's own key-switch pieces (Alloc_precomp, Dot_prod, Mod_down, Rescale, Automorphism_transform of
    the compiled reference, oracle/_ref/ref_driver) at this level on this host, one thread, each run once on uniform
    residues; None where that binary is absent."""
    import refdrv

    if not refdrv.available():
        return None
    s = refdrv.RefSession(*CFG)
    k = s.add(refdrv.OP_TIME_KEYSWITCH, level, 7)
    _, res = s.run()
    pre, dot, down, resc, auto = (int(v) * 1e-9 for v in res[k])
    note = "the reference's Alloc_precomp / 2 x Dot_prod / 2 x Mod_down / 2 x Rescale / 2 x Automorphism_transform, once each, gcc -O3"
    return {"keyswitch_cpu_baseline": {"s_per_op": round(pre + dot + down + resc, 3), "cores": 1, "kind": "reference",
                                       "parts_s": {"precomp": round(pre, 3), "dot_prod_x2": round(dot, 3),
                                                   "mod_down_x2": round(down, 3), "rescale_x2": round(resc, 3)},
                                       "sample": note},
            "rotation_cpu_baseline": {"s_per_rotation": round(dot + down + auto, 3), "hoisted_precomp_s": round(pre, 3),
                                      "cores": 1, "kind": "reference", "sample": note}}


def extra_legs(g, which="all"):
    import headline
    from oracle_lib import Oracle

    level = g.L
    o = Oracle(*CFG)  # the checker of one operation per leg, outside the timed regions
    swk_host = headline.seeded_key(g.primes)
    cts_host = headline.seeded_ciphertexts(g.primes, level)
    swk = g.upload(swk_host)
    cts = [g.upload(c) for c in cts_host]
    extra = {}
    if which in ("all", "keyswitch"):
        extra.update(keyswitch_leg(g, o, swk_host, cts_host, swk, cts))
    if which in ("all", "rotation"):
        extra.update(rotation_leg(g, o, swk_host, cts_host, swk, cts))
    o.close()
    for b in cts + [swk]:
        b.free()
    ref = keyswitch_cpu_reference(level)
    if ref:
        if "keyswitch_ops_per_s" in extra:
            extra["keyswitch_cpu_baseline"] = ref["keyswitch_cpu_baseline"]
        if "rotations_per_s" in extra:
            extra["rotation_cpu_baseline"] = ref["rotation_cpu_baseline"]
    return extra


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="time budget of the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the key-switch / rotation measurements")
    ap.add_argument("--only-extra", choices=("all", "keyswitch", "rotation"), default=None,
                    help="profiling aid: run only the key-switch and/or rotation legs (prints their fields alone)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU; this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np

    import acefhe
    import seeded

    g = acefhe.Context(*CFG)
    if not g.has_device:
        log("no GPU visible: " + g.err())
        sys.exit(1)
    assert (g.L, g.K, g.part_size) == (24, 7, 8)
    idx = list(range(LIMBS))
    per_poly = LIMBS * N
    log("generating %d x %d limbs of seeded input" % (POLYS, LIMBS))
    x_host = np.concatenate([seeded.uniform_poly(1000 + p, g.primes[:LIMBS], N) for p in range(POLYS)])
    x = g.upload(x_host)

    def step():
        g.ntt(x, x, idx, n_polys=POLYS, poly_stride_limbs=LIMBS)
        g.intt(x, x, idx, n_polys=POLYS, poly_stride_limbs=LIMBS)

    if args.only_extra:
        args.warmup, args.steps = 0, 1
    else:
        settle(g, step)  # untimed, before the warm-up steps: see settle()
    for _ in range(args.warmup):
        step()
    g.sync()
    t0 = time.perf_counter()
    g.timer_start()
    for _ in range(args.steps):
        step()
    ev_ms = g.timer_stop_ms()
    g.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = wall_ms / args.steps
    assert (x.get() == x_host).all(), "round trip did not return the input"
    # the forward half on its own: one polynomial of the batch, transformed with the batch, against the oracle
    from oracle_lib import Oracle

    o = Oracle(*CFG)
    g.ntt(x, x, idx, n_polys=POLYS, poly_stride_limbs=LIMBS)
    p = 19
    fwd_ok = bool((x.view(p * per_poly, per_poly).get() == o.ntt(x_host[p * per_poly:(p + 1) * per_poly], idx)).all())
    o.close()
    assert fwd_ok, "forward NTT of polynomial %d of the batch differs from the oracle" % p
    g.intt(x, x, idx, n_polys=POLYS, poly_stride_limbs=LIMBS)
    step_bytes = POLYS * per_poly * 16 * 2
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # per-kernel timing of the four NTT kernels (each reads and writes every coefficient once)
    kern = {}
    if args.only_extra:
        print(json.dumps(extra_legs(g, args.only_extra)))
        return
    scratch = g.alloc(POLYS * per_poly)
    pass_bytes = POLYS * per_poly * 16
    # a plain device copy of the whole batch: the known-size kernel against which the
    # FETCH_SIZE / WRITE_SIZE counters of a profiling run are calibrated
    g.copy(scratch, x)
    g.sync()
    # (the names are those of the kernels these four passes launch on this workload)
    for name, inv, which in (("ntt_fwd_strided", 0, 1), ("ntt_fwd_chunk_run", 0, 2), ("ntt_inv_half_run", 1, 1),
                             ("ntt_inv_strided", 1, 2)):
        src = x if which == 1 else scratch
        f = lambda: g.ntt_pass(scratch, src, idx, POLYS, LIMBS, inv, which)
        f()
        ms = time_region(g, f, 20)
        kern[name] = {"ms": round(ms, 4), "GB/s": round(pass_bytes / (ms * 1e-3) / 1e9, 1)}
    dom = max(kern, key=lambda k: kern[k]["ms"])
    roofline = {"bound": "hbm", "kernel": dom, "achieved": kern[dom]["GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(kern[dom]["GB/s"] / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_BYTES.get(dom),
                "bytes_per_launch": pass_bytes, "all_ntt_kernels": kern}
    scratch.free()

    extra = {} if args.no_extra else extra_legs(g)
    if not args.no_extra:
        extra.update(bootstrap_leg())
        extra.update(resnet20_leg())

    cpu = cpu_baseline(x_host, idx, args.cpu_seconds) if args.cpu_seconds > 0 else None

    out = {
        "metric": "ntt_roundtrip_algorithmic_bandwidth", "value": round(value, 2), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u64", "data": "synthetic",
        "config": {"workload": "batched RNS NTT+INTT round trip, 32 polys x 24 limbs (50-bit primes), N=65536",
                   "bytes_per_step": step_bytes, "hbm_frac": round(value / HBM_PEAK_GBS, 4),
                   "event_ms_per_step": round(ev_ms / args.steps, 4), "forward_verified": fwd_ok},
        "roofline": roofline, "cpu_baseline": cpu, "extra": extra,
    }
    print(json.dumps(out))
    g.close()


if __name__ == "__main__":
    main()
