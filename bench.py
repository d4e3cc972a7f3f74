#!/usr/bin/env python3
"""Benchmark of the MI355X zkLLM prover core.

One step = one LLaMa-2-7B-shape decoder layer at sequence length 2048, computed and proved end to end on one
GPU with weights, generators, commitments and the input already resident in HBM: RMSNorm x2, Q/K/V/O
projections, 32 attention heads (QK^T, zkSoftmax, YV), SwiGLU FFN, every rescaling / lookup / sumcheck and
the opening of all nine weight commitments.  `value` is seconds per layer.

The same JSON line also carries the two throughput figures of the headline metric (G1 MSM points/s on the
4096 x 11008 commitment workload, Fr multiplications/s), a roofline entry for the kernel with the largest share
of the layer's GPU time (timed with HIP events around its launches inside the timed region), roofline entries of
the generic Fr matmul and of an HBM-bound fold, and a CPU baseline measured with the oracle on this host's cores.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
# VALU integer peak: 256 CUs x 4 SIMDs x 16 lanes x 2.4 GHz lane-operations per second (v_mad_u64_u32 issues at
# full rate on gfx950; bench measures it as well and reports the measured figure next to this one)
VALU_PEAK_TOPS = 256 * 4 * 16 * 2.4e9 / 1e12
# HBM traffic of k_open_fold per generator pair, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on the kernel alone
# (python3 bench.py --pmc-probe; summary in profiles/k_open_fold_pmc_traffic.txt), each counter scaled by what it reads for
# zk_fr_add over 2^24 elements (1 GiB read, 512 MiB written)
FOLD_TRAFFIC_BYTES_PER_PAIR = 2551.0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--seq", type=int, default=2048)
    ap.add_argument("--head-group", type=int, default=32,
                    help="attention proved this many heads at a time with zkAttnStacked (a divisor of 32; default: all 32 as one stack); "
                         "0 = head by head, the flow of self-attn.cu per head")
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--skip-extras", action="store_true", help="only the layer timing (used for profiling runs)")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="for rocprofv3 --pmc runs: only three launches of the opening's fold kernel at 262144 pairs and one "
                         "zk_fr_add over 2^24 elements (1 GiB read, 512 MiB written) to scale the counters by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this prover runs on one GPU; every configuration of the benchmark fits a single MI355X, "
              "so --gpus must be 1 (no multi-GPU path exists in this build)", file=sys.stderr)
        sys.exit(2)

    from gpuhelp import Hip, Prover, c_int, c_size_t, c_uint, c_void_p
    import layercfg
    from zkhelp import mt_random_vec

    pv = Prover()
    hip = Hip()
    lib = hip.lib

    if args.pmc_probe:
        n_big = 1 << 19
        pv.seed(6)
        gens_big = pv.commitment_random(n_big)
        pv.lib.zkp_g1_devptr.restype = ctypes.c_void_p
        gp = pv.lib.zkp_g1_devptr(c_void_p(gens_big.h))
        sc = hip.upload(mt_random_vec(np.random.RandomState(8), n_big))
        ns, ng = hip.malloc(32 * (n_big // 2)), hip.malloc(144 * (n_big // 2))
        u1 = mt_random_vec(np.random.RandomState(9), 1)
        sums3 = np.zeros((3, 36), np.uint32)
        for _ in range(3):
            hip.call("zk_g1_open_round", c_void_p(ns), c_void_p(ng), sums3, c_void_p(sc), c_void_p(gp), u1, c_size_t(n_big), None)
        n = 1 << 24
        dA, dB, dO = hip.malloc(32 * n), hip.malloc(32 * n), hip.malloc(32 * n)
        hip.call("zk_fr_add", c_void_p(dO), c_void_p(dA), c_void_p(dB), c_size_t(n), None)
        # the kernels behind the other reported rates, once each on operands of known size: the Montgomery product
        # (Fr mul/s), the fused three-level fold (HBM GB/s) and the commitment of the 11008 x 4096 weight (MSM points/s)
        seed_block = mt_random_vec(np.random.RandomState(1), 1 << 16)
        src = hip.upload(seed_block)
        for i in range(n >> 16):
            lib.zk_memcpy_d2d(c_void_p(dA + i * (32 << 16)), c_void_p(src), c_size_t(32 << 16), None)
            lib.zk_memcpy_d2d(c_void_p(dB + i * (32 << 16)), c_void_p(src + 32 * 5), c_size_t((32 << 16) - 32 * 5), None)
        hip.call("zk_fr_montmul", c_void_p(dO), c_void_p(dA), c_void_p(dB), c_size_t(n), None)
        u3 = mt_random_vec(np.random.RandomState(2), 3)
        hip.call("zk_fr_fold_axis", c_void_p(dO), c_void_p(dA), u3, c_int(3), c_size_t(1), c_uint(2048), c_size_t(4096), None)
        pv.seed(5)
        gens = pv.commitment_random(4096)
        Wm = np.round(np.random.default_rng(12).normal(0, 0.02, (11008, 4096)) * 65536).astype(np.int32)
        com = pv.commit_int(gens, pv.from_i32(Wm))
        hip.sync()
        print(json.dumps({"pmc_probe": {"fold_pairs_per_launch": n_big // 2, "fold_launches": 3, "copy_kernel": "k_ew<0> (zk_fr_add)",
                                        "copy_read_bytes": 64 * n, "copy_write_bytes": 32 * n, "montmul_elements": n,
                                        "fold_axis_elements_in": 2048 * 4096, "msm_pairs": 11008 * 4096}}))
        return

    def ev():
        e = c_void_p()
        hip.check(lib.zk_event_create(ctypes.byref(e)))
        return e

    def time_kernel(fn, reps, warm=1):
        """average duration in ms of `fn` (one launch on the default stream), HIP events on that stream"""
        for _ in range(warm):
            fn()
        e0, e1 = ev(), ev()
        hip.check(lib.zk_event_record(e0, None))
        for _ in range(reps):
            fn()
        hip.check(lib.zk_event_record(e1, None))
        ms = ctypes.c_float()
        hip.check(lib.zk_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
        return ms.value / reps

    # ---- workload: the decoder layer ------------------------------------------------------------------------------
    seq = args.seq
    cu, cf = layercfg.llama7b(seq=seq, open_weights=True, head_group=args.head_group)
    t0 = time.perf_counter()
    pv.seed(2024)
    layer = pv.layer_create_random(cu, cf, 7, 5)
    pv.sync()
    setup_s = time.perf_counter() - t0
    X = np.round(np.random.default_rng(11).normal(0, 1, (seq, 4096)) * 65536).astype(np.int32)
    hX = pv.from_i32(X)
    devnull = os.open(os.devnull, os.O_WRONLY)
    saved_stdout = os.dup(1)
    os.dup2(devnull, 1)      # the class layer prints the reference's progress lines ("Opening complete", ...)
    try:
        parts = np.zeros(8)
        for _ in range(args.warmup):
            pv.layer_run(layer, hX)
        pv.sync()
        hip.check(lib.zk_prof_fold_begin())
        t0 = time.perf_counter()
        for _ in range(args.steps):
            _, times = pv.layer_run(layer, hX)
            parts += times
        pv.sync()
        wall = time.perf_counter() - t0
        fold_ms, fold_launches, fold_mults, fold_pairs = ctypes.c_double(), ctypes.c_ulonglong(), ctypes.c_double(), ctypes.c_ulonglong()
        hip.check(lib.zk_prof_fold_read(ctypes.byref(fold_ms), ctypes.byref(fold_launches), ctypes.byref(fold_mults), ctypes.byref(fold_pairs)))
    finally:
        os.dup2(saved_stdout, 1)
    ms_per_step = wall * 1e3 / args.steps
    parts /= args.steps
    live_b, cached_b = ctypes.c_size_t(), ctypes.c_size_t()
    hip.check(lib.zk_pool_stats(ctypes.byref(live_b), ctypes.byref(cached_b)))
    pool_gib = (live_b.value + cached_b.value) / 2 ** 30      # the allocator keeps what it once needed: live + cached = the layer's peak
    pv.layer_free(layer)
    lib.zk_pool_trim()

    out = {
        "metric": "layer prove time (s), 7B shape seq 2048; G1 MSM points/s; Fr mul/s",
        "value": ms_per_step / 1e3,
        "unit": "s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u32",
        "data": "synthetic",
        "config": {"workload": f"C5: LLaMa-2-7B-shape decoder layer proof, seq {seq}, hidden 4096, 32 heads x 128, FFN 11008, "
                               "random-init fixed-point weights (scale 2^16), generators of size out_features<<5, all nine weight openings included; attention proved "
                               + (f"{args.head_group} heads at a time as head-major stacks (zkAttnStacked)" if args.head_group else "head by head"),
                   "device_pool_gib": round(pool_gib, 1),
                   "setup_s_untimed": round(setup_s, 3),
                   "parts_ms": {k: round(float(v), 1) for k, v in zip(["rmsnorm1", "qkv", "attention", "oproj", "rmsnorm2", "ffn", "total", "open_wait"], parts)}},
    }
    # roofline of the kernel with the largest share of the layer's GPU time: the generator fold of the openings
    # (one endomorphism-split scalar multiplication per pair).  It is bound by 32-bit integer multiply-adds: an
    # Fp multiplication is 2*12^2+12 = 300 of them.  Durations are HIP events around every launch inside the timed
    # region above, on the launch stream.
    MAD_PER_FP_MUL = 300
    fold_tops = fold_mults.value * MAD_PER_FP_MUL / (fold_ms.value * 1e-3) / 1e12 if fold_ms.value > 0 else 0.0
    out["roofline"] = {"kernel": "k_open_fold (opening: g' = g1 + [u](g0 - g1) per pair, 128-bit split scalars)", "bound": "valu-int",
                       "achieved": fold_tops, "peak": VALU_PEAK_TOPS, "unit": "T MAD32/s", "frac": fold_tops / VALU_PEAK_TOPS,
                       "traffic": FOLD_TRAFFIC_BYTES_PER_PAIR * fold_pairs.value / max(1, fold_launches.value),
                       "launches": int(fold_launches.value), "avg_launch_ms": fold_ms.value / max(1, fold_launches.value),
                       "total_ms_in_timed_region": fold_ms.value, "pairs": int(fold_pairs.value), "fp_mul_per_s": fold_mults.value / (fold_ms.value * 1e-3) if fold_ms.value > 0 else 0.0,
                       "note": "algorithmic work = Fp multiplications of the point formulas x 300 MAD32 (12-limb schoolbook product and reduction; the kernel "
                               "itself works on 14 limbs of 29 bits: 392 multiply-adds and ~110 other instructions per product, 301 per square); "
                               "peak = 256 CU x 4 SIMD x 16 lanes x 2.4 GHz.  traffic = measured bytes per pair (rocprofv3 FETCH_SIZE + WRITE_SIZE of the kernel alone, "
                               "profiles/k_open_fold_pmc_traffic.txt) x the average pairs per launch; algorithmic traffic is 336 B per pair.  The average covers every "
                               "launch of the timed region: most are short rounds (one wave per SIMD or less) that run beside the rest of the proof"}
    if args.skip_extras:
        print(json.dumps(out))
        return

    # ---- the same fold kernel alone at its largest shape in the layer: one halving of 2^19 generators (the FFN weights' opening) ----
    pv.seed(6)
    n_big = 1 << 19
    gens_big = pv.commitment_random(n_big)
    pv.lib.zkp_g1_devptr.restype = ctypes.c_void_p
    gp = pv.lib.zkp_g1_devptr(c_void_p(gens_big.h))
    sc = hip.upload(mt_random_vec(np.random.RandomState(8), n_big))
    ns, ng = hip.malloc(32 * (n_big // 2)), hip.malloc(144 * (n_big // 2))
    u1 = mt_random_vec(np.random.RandomState(9), 1)
    sums3 = np.zeros((3, 36), np.uint32)
    hip.call("zk_g1_open_round", c_void_p(ns), c_void_p(ng), sums3, c_void_p(sc), c_void_p(gp), u1, c_size_t(n_big), None)
    hip.check(lib.zk_prof_fold_begin())
    for _ in range(3):
        hip.call("zk_g1_open_round", c_void_p(ns), c_void_p(ng), sums3, c_void_p(sc), c_void_p(gp), u1, c_size_t(n_big), None)
    hip.check(lib.zk_prof_fold_read(ctypes.byref(fold_ms), ctypes.byref(fold_launches), ctypes.byref(fold_mults), ctypes.byref(fold_pairs)))
    iso_tops = fold_mults.value * MAD_PER_FP_MUL / (fold_ms.value * 1e-3) / 1e12
    out["roofline_fold_alone"] = {"kernel": "k_open_fold, 262144 pairs, nothing else on the device", "bound": "valu-int", "achieved": iso_tops, "peak": VALU_PEAK_TOPS,
                                  "unit": "T MAD32/s", "frac": iso_tops / VALU_PEAK_TOPS, "traffic": FOLD_TRAFFIC_BYTES_PER_PAIR * (n_big // 2),
                                  "avg_launch_ms": fold_ms.value / max(1, fold_launches.value),
                                  "fp_mul_per_s": fold_mults.value / (fold_ms.value * 1e-3),
                                  "note": "4096 waves on 2048 wave slots (two per SIMD: 250 registers, most of the walk's table in LDS): two full turns.  traffic: FETCH_SIZE + "
                                          "WRITE_SIZE of this launch from profiles/k_open_fold_pmc_traffic.txt, against 336 B per pair of algorithmic traffic (the rest is "
                                          "private memory of the out-of-line special cases)"}
    for p_ in (sc, ns, ng):
        hip.free(p_)
    del gens_big

    # ---- G1 MSM points/s: commitment of a 4096 x 11008 weight (stored 11008 rows x 4096 against 4096 generators) -------------
    pv.seed(5)
    gens = pv.commitment_random(4096)
    Wm = np.round(np.random.default_rng(12).normal(0, 0.02, (11008, 4096)) * 65536).astype(np.int32)
    hW = pv.from_i32(Wm)
    pv.commit_int(gens, hW)
    pv.sync()
    t0 = time.perf_counter()
    reps = 3
    for _ in range(reps):
        com = pv.commit_int(gens, hW)
    pv.sync()
    msm_s = (time.perf_counter() - t0) / reps
    out["g1_msm_points_per_s"] = 11008 * 4096 / msm_s
    out["g1_msm_ms"] = msm_s * 1e3
    del com, hW, gens

    # ---- Fr mul/s: n independent Montgomery products on resident operands ------------------------------------------------------
    n = 1 << 26
    seed_block = mt_random_vec(np.random.RandomState(1), 1 << 16)
    src = hip.upload(seed_block)
    dA, dB, dO = hip.malloc(32 * n), hip.malloc(32 * n), hip.malloc(32 * n)
    for i in range(n >> 16):
        lib.zk_memcpy_d2d(c_void_p(dA + i * (32 << 16)), c_void_p(src), c_size_t(32 << 16), None)
        lib.zk_memcpy_d2d(c_void_p(dB + i * (32 << 16)), c_void_p(src + 32 * 5), c_size_t((32 << 16) - 32 * 5), None)
    hip.sync()
    mul_ms = time_kernel(lambda: hip.call("zk_fr_montmul", c_void_p(dO), c_void_p(dA), c_void_p(dB), c_size_t(n), None), reps=10)
    add_ms = time_kernel(lambda: hip.call("zk_fr_add", c_void_p(dO), c_void_p(dA), c_void_p(dB), c_size_t(n), None), reps=10)
    out["fr_mul_per_s"] = n / (mul_ms * 1e-3)
    out["fr_mul_stream_gbs"] = 96 * n / (mul_ms * 1e-3) / 1e9
    out["fr_add_stream_gbs"] = 96 * n / (add_ms * 1e-3) / 1e9

    # measured VALU multiply-add peak
    peak = ctypes.c_double()
    hip.check(lib.zk_bench_mad_peak(c_uint(256 * 32), c_uint(10000), ctypes.byref(peak), None))
    out["valu_mad32_peak_measured_tops"] = peak.value / 1e12

    # ---- roofline of the kernels that dominate the layer ---------------------------------------------------------------------------
    # (1) generic Fr matmul at the projection shape: M*N*P field multiplications, 136 MAD32 each (algorithmic)
    M, N, P = 2048, 4096, 4096
    mm_ms = time_kernel(lambda: hip.call("zk_fr_matmul_generic", c_void_p(dO), c_void_p(dA), c_void_p(dB), c_uint(M), c_uint(N), c_uint(P), None), reps=1)
    # (2) fused multilinear fold (3 levels per pass) over a 2048 x 4096 tensor: 32 B read per element
    u = mt_random_vec(np.random.RandomState(2), 3)
    fold_ms = time_kernel(lambda: hip.call("zk_fr_fold_axis", c_void_p(dO), c_void_p(dA), u, c_int(3), c_size_t(1), c_uint(2048), c_size_t(4096), None), reps=10)
    fold_gbs = 32 * 2048 * 4096 / (fold_ms * 1e-3) / 1e9
    mm_tops = M * N * P * 72 / (mm_ms * 1e-3) / 1e12
    out["roofline_matmul"] = {"kernel": "k_matmul (generic Montgomery Fr matmul, 2048x4096x4096)", "bound": "valu-int", "achieved": mm_tops, "peak": VALU_PEAK_TOPS,
                              "unit": "T MAD32/s", "frac": mm_tops / VALU_PEAK_TOPS, "traffic": None,
                              "note": "algorithmic 72 MAD32 per field multiply-accumulate (64 limb products + 1/8 of a shared reduction); every MAD32 needs a second "
                                      "VALU instruction for its carry, so 0.5 is the ceiling of this formulation",
                              "avg_launch_ms": mm_ms, "gmac_per_s": M * N * P / (mm_ms * 1e-3) / 1e9}
    out["roofline_hbm"] = {"kernel": "k_fold_axis_dot<3> (fused 3-level multilinear fold, 2048x4096)", "bound": "hbm", "achieved": fold_gbs, "peak": HBM_PEAK_GBS,
                           "unit": "GB/s", "frac": fold_gbs / HBM_PEAK_GBS, "traffic": None, "avg_launch_ms": fold_ms}
    for p in (dA, dB, dO, src):
        hip.free(p)

    # ---- CPU baseline: the oracle's restatement of the reference's algorithm on this host's cores ---------------------------------------
    # A bounded sample of the two costs that dominate the reference's layer: the field multiplications of the matrix products
    # and the five 255-bit scalar multiplications per generator pair of the openings; both scaled to the layer's counts.
    if not args.skip_cpu:
        from zkhelp import load_oracle
        orc = load_oracle()
        cores = orc.dll.orc_num_threads()
        B = mt_random_vec(np.random.RandomState(4), 4096 * 1024)

        def mm_sample(rows):
            A = mt_random_vec(np.random.RandomState(3), rows * 4096)
            C = np.zeros((rows * 1024, 8), np.uint32)
            t0 = time.perf_counter()
            orc.orc_fr_matmul_rows(A, B, rows, 4096, 1024, rows, C)
            return time.perf_counter() - t0
        probe_rows = 2 * max(1, cores // 2)
        dt = mm_sample(probe_rows)
        rows = int(max(probe_rows, min(4096, probe_rows * 20.0 / max(dt, 1e-3)))) // max(1, cores) * max(1, cores)
        rows = max(rows, probe_rows)
        dt = mm_sample(rows)
        mm_rate = rows * 4096 * 1024 / dt                      # field multiplications per second, all cores
        # opening sample: n generators, one row
        n_open = 4096
        gens = np.zeros((n_open, 36), np.uint32)
        orc.orc_seed(99)
        gens = np.zeros((n_open, 36), np.uint32)
        orc.orc_commitment_random(n_open, gens)
        T = mt_random_vec(np.random.RandomState(6), n_open)
        k = 12
        u = mt_random_vec(np.random.RandomState(7), k)
        proof = np.zeros((3 * k + 1, 36), np.uint32)
        val = np.zeros(8, np.uint32)
        t0 = time.perf_counter()
        orc.orc_open(gens, n_open, T, n_open, 1, u, k, proof, val)
        open_s = time.perf_counter() - t0
        layer_mm = 4.49e11                                     # field multiplications in the layer's matrix products (reference algorithm)
        layer_gens = 5 * (4096 << 5) + 2 * (1 << 19) + 2 * 4096      # generators of the nine openings (11008 << 5 rounds up to 2^19); pairs over all rounds ~ the same number
        cpu_s = layer_mm / mm_rate + open_s * layer_gens / n_open
        out["cpu_baseline"] = {"value": cpu_s, "unit": "s", "cores": int(cores), "kind": "port",
                               "sample": f"oracle (reference algorithm, OpenMP): Fr matmul {rows} x 4096 x 1024 = {rows * 4096 * 1024:.3g} multiplications in {dt:.1f} s, "
                                         f"scaled to the layer's 4.49e11; opening of {n_open} generators in {open_s:.1f} s, scaled to the layer's "
                                         f"{layer_gens} generators; sumchecks and lookups not included (lower bound of the CPU layer time)",
                               "fr_mul_per_s_all_cores": mm_rate}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
