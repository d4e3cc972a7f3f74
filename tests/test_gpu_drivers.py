"""The per-block executables (ppgen, commit-param, rmsnorm, self-attn, ffn, skip-connection) run as child processes over
.bin files, with the argument lists and file names that the reference's llama-*.py scripts use: every file they write is
compared byte for byte with the CPU oracle's result for the same block, and every proof file (field transcript and the
opening points) with the oracle's transcript under the same seed."""
import os
import struct
import subprocess

import numpy as np
import pytest

import layercfg
from zkhelp import FP_R, P_MOD, R_MOD, ROOT, fr_array, fr_signed, jac_to_affine, load_oracle, orc_check, orc_transcript, to_limbs

pytestmark = pytest.mark.gpu

BIN = os.path.join(ROOT, "zkllm-ccs2024_amd", "host")
TINY_ENV = "sf_linear=256,sf_gate=1024,sf_attn=128,softmax_bs=256:256:256,softmax_L=1,softmax_M=0,softmax_sf_in=65536,softmax_thetas=64:256,value_scale=256"
LOF = 1            # log_off_factor of llama-ppgen.py (generators per 2-D weight = out_features << LOF)


def exe(name):
    path = os.path.join(BIN, name)
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build the executables with `make -C zkllm-ccs2024_amd/host drivers-all` (or __graft_entry__.build())")
    return path


def run(cwd, seed, proof, *argv, config=TINY_ENV, extra_env=None):
    env = dict(os.environ, ZKLLM_SEED=str(seed))
    if config:
        env["ZKLLM_LAYER_CONFIG"] = config
    if proof:
        env["ZKLLM_PROOF_FILE"] = str(proof)
    env.update(extra_env or {})
    print("run", " ".join(str(a) for a in argv), "seed", seed, flush=True)
    r = subprocess.run([exe(argv[0])] + [str(a) for a in argv[1:]], cwd=str(cwd), env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, f"{argv[0]} failed ({r.returncode}): {r.stdout[-2000:]} {r.stderr[-2000:]}"
    return r.stdout


def read_proof(path):
    raw = open(path, "rb").read()
    assert raw[:8] == b"ZKLLMPF1"
    n_fr, n_g1 = struct.unpack("<QQ", raw[8:24])
    assert len(raw) == 24 + 32 * n_fr + 144 * n_g1
    fr = np.frombuffer(raw, dtype=np.uint32, count=8 * n_fr, offset=24).reshape(n_fr, 8)
    g1 = np.frombuffer(raw, dtype=np.uint32, count=36 * n_g1, offset=24 + 32 * n_fr).reshape(n_g1, 36)
    return fr, g1


def normalise(points):
    """Jacobian rows -> the canonical rows (x / z^2, y / z^3, ONE) in Montgomery form, infinity as zero limbs (python big integers)"""
    out = np.zeros((len(points), 36), np.uint32)
    for i, row in enumerate(np.asarray(points, dtype=np.uint32).reshape(-1, 36)):
        P = jac_to_affine(row)
        if P is not None:
            out[i] = to_limbs(P[0] * FP_R % P_MOD, 12) + to_limbs(P[1] * FP_R % P_MOD, 12) + to_limbs(FP_R, 12)
    return out


def g1_file(path):
    return np.fromfile(path, dtype=np.uint32).reshape(-1, 36)


def as_fr(a):
    return fr_array([int(x) % R_MOD for x in np.asarray(a).reshape(-1)])


def fr_to_i64(fr):
    return np.array(fr_signed(fr), dtype=np.int64)


class OracleWeight:
    def __init__(self, orc, w, in_dim, out_dim, gens, com):
        import ctypes
        orc.dll.orc_weight_new.restype = ctypes.c_void_p
        self.orc = orc
        h = orc.orc_weight_new(np.ascontiguousarray(w, dtype=np.int32), in_dim, out_dim, np.ascontiguousarray(gens), len(gens), np.ascontiguousarray(com), len(com))
        assert h, orc.dll.orc_last_error()
        self.h = ctypes.c_void_p(h)

    def __del__(self):
        self.orc.orc_weight_free(self.h)


def check_proof(orc, path, seed_note):
    fr, g1 = read_proof(path)
    exp = orc_transcript(orc)
    assert fr.shape == exp.shape and (fr == exp).all(), seed_note
    n = orc.dll.orc_g1_transcript_size()
    raw = np.zeros((n, 36), np.uint32)
    if n:
        orc.orc_g1_transcript_get(raw)
    assert g1.shape == (n, 36) and (g1 == normalise(raw)).all(), seed_note
    return fr.shape[0], n


def test_executables_chain_over_bin_files_matches_the_oracle_byte_for_byte(tmp_path):
    orc = load_oracle()
    orc.dll.orc_g1_transcript_size.restype = __import__("ctypes").c_long
    cu, cf = layercfg.tiny(open_weights=True)
    S, E, Hd = int(cu[0]), int(cu[1]), int(cu[3])
    ws = layercfg.tiny_weights(21, cu)
    names = ["input_layernorm.weight", "self_attn.q_proj.weight", "self_attn.k_proj.weight", "self_attn.v_proj.weight", "self_attn.o_proj.weight",
             "post_attention_layernorm.weight", "mlp.up_proj.weight", "mlp.gate_proj.weight", "mlp.down_proj.weight"]
    work = tmp_path / "zkllm-workdir"
    work.mkdir()
    prefix = "layer-0"
    X = np.round(np.random.default_rng(31).normal(0, 1, (S, E)) * 256).astype(np.int32)
    X.tofile(tmp_path / "layer_input.bin")

    # ---- llama-ppgen.py / llama-commit.py: generators and commitments of every parameter ------------------------------------
    seed = 100
    W = {}
    for name, w in zip(names, ws):
        one_d = name.endswith("layernorm.weight")
        in_dim, out_dim = (w.shape[1], 1) if one_d else w.shape           # llama-commit.py passes (len, 1) for 1-D parameters
        pp_size = w.shape[1] if one_d else (w.shape[1] << LOF)            # HF shape[0] = out_features
        pp, ib, cb = work / f"{name}-pp.bin", work / f"{prefix}-{name}-int.bin", work / f"{prefix}-{name}-commitment.bin"
        seed += 1
        run(tmp_path, seed, None, "ppgen", pp_size, pp, config=None)
        n_gen = 1 << (pp_size - 1).bit_length()
        orc.orc_seed(seed)
        e_gens = np.zeros((n_gen, 36), np.uint32)
        orc_check(orc.orc_commitment_random(n_gen, e_gens))
        gens = g1_file(pp)
        assert gens.shape == (n_gen, 36) and (gens == normalise(e_gens)).all(), name      # z = ONE: byte-identical to the double-and-add path
        w.astype(np.int32).tofile(ib)
        out = run(tmp_path, seed, None, "commit-param", pp, ib, cb, in_dim, out_dim, config=None)
        com = g1_file(cb)
        rows_p, cols_p = 1 << (in_dim - 1).bit_length(), 1 << (out_dim - 1).bit_length()
        padded = np.zeros((rows_p, cols_p), np.int64)
        padded[:in_dim, :out_dim] = w.reshape(in_dim, out_dim)
        e_com = np.zeros((padded.size // n_gen, 36), np.uint32)
        orc_check(orc.orc_commit_int(gens, n_gen, as_fr(padded), padded.size, e_com))
        assert com.shape == e_com.shape and (com == normalise(e_com)).all(), name        # MSM path == commit_int_dev_func path, byte for byte
        assert f"Commitment size: {com.shape[0]}" in out
        # the blocks open the norm weights as 1 x E (rmsnorm.cu:19-24), the others as in x out
        W[name] = OracleWeight(orc, w, 1 if one_d else in_dim, w.shape[1] if one_d else out_dim, gens, com)

    def rms_inv_file(x_int):
        """llama-rmsnorm.py:35-39"""
        xf = x_int.astype(np.float64) / 256.0
        r = np.rint(1.0 / np.sqrt(np.mean(xf ** 2, axis=1) + 1e-5) * 256.0).astype(np.int32)
        r.tofile(tmp_path / "rms_inv_temp.bin")
        return r

    def block(seed, proof_name, argv, oracle_call):
        proof = tmp_path / proof_name
        run(tmp_path, seed, proof, *argv)
        orc.orc_seed(seed)
        orc.orc_transcript_clear()
        oracle_call()
        return check_proof(orc, proof, proof_name)

    # ---- rmsnorm input ------------------------------------------------------------------------------------------------------------
    rms = rms_inv_file(X)
    e_out = np.zeros((S * E, 8), np.uint32)
    n_fr, n_g1 = block(201, "rmsnorm1.proof", ["rmsnorm", "input", "layer_input.bin", S, E, work, prefix, "attn_input.bin"],
                       lambda: orc_check(orc.orc_rmsnorm_block(cu, cf, W[names[0]].h, as_fr(X), as_fr(rms), e_out)))
    a_in = np.fromfile(tmp_path / "attn_input.bin", dtype=np.int32)
    assert (a_in == fr_to_i64(e_out)).all() and n_fr > 50 and n_g1 == 3 * 5 + 1          # 32 generators: 5 halving rounds
    # ---- self-attn linear ---------------------------------------------------------------------------------------------------------
    eQ, eK, eV = (np.zeros((S * E, 8), np.uint32) for _ in range(3))
    n_fr, n_g1 = block(202, "linear.proof", ["self-attn", "linear", "attn_input.bin", S, E, work, prefix, "attn_output.bin"],
                       lambda: orc_check(orc.orc_attn_linear_block(cu, cf, W[names[1]].h, W[names[2]].h, W[names[3]].h, as_fr(a_in), eQ, eK, eV)))
    Q, K, V = (np.fromfile(tmp_path / f"temp_{n}.bin", dtype=np.int32) for n in "QKV")
    assert (Q == fr_to_i64(eQ)).all() and (K == fr_to_i64(eK)).all() and (V == fr_to_i64(eV)).all()
    assert n_g1 == 3 * (3 * 6 + 1)                                                       # three openings over 64 generators
    # ---- self-attn attn: one head as wide as the tensors, as the reference's executable does it --------------------------------
    e_att, e_Y = np.zeros((S * E, 8), np.uint32), np.zeros((S * S, 8), np.uint32)
    block(203, "attn.proof", ["self-attn", "attn", "attn_input.bin", S, E, work, prefix, "attn_output.bin"],
          lambda: orc_check(orc.orc_attn_block(cu, cf, 1, as_fr(Q), as_fr(K), as_fr(V), e_att, e_Y)))
    head_out = np.fromfile(tmp_path / "temp_head_out.bin", dtype=np.int32)
    assert (head_out == fr_to_i64(e_att)).all()
    assert (np.fromfile(tmp_path / "temp_head_Y.bin", dtype=np.int64) == fr_to_i64(e_Y)).all()
    assert not (tmp_path / "attn_output.bin").exists()                                   # the reference's attn mode leaves its output argument alone
    # ---- skip connection, second norm ------------------------------------------------------------------------------------------
    run(tmp_path, 204, None, "skip-connection", "layer_input.bin", "temp_head_out.bin", "attn_output.bin")
    x2 = np.fromfile(tmp_path / "attn_output.bin", dtype=np.int32)
    assert (x2 == X.reshape(-1) + head_out).all()
    rms2 = rms_inv_file(x2.reshape(S, E))
    block(205, "rmsnorm2.proof", ["rmsnorm", "post_attention", "attn_output.bin", S, E, work, prefix, "ffn_input.bin"],
          lambda: orc_check(orc.orc_rmsnorm_block(cu, cf, W[names[5]].h, as_fr(x2), as_fr(rms2), e_out)))
    f_in = np.fromfile(tmp_path / "ffn_input.bin", dtype=np.int32)
    assert (f_in == fr_to_i64(e_out)).all()
    # ---- ffn: the output file holds the down projection before its rescaling (ffn.cu:81) -----------------------------------------
    table = np.zeros((int(cu[9]), 8), np.uint32)
    orc_check(orc.orc_swiglu_table(int(cf[1]), int(cu[9]), cf[2], cf[3], table))
    fr_to_i64(table).astype(np.int32).tofile(tmp_path / "swiglu-table.bin")
    e_down = np.zeros((S * E, 8), np.uint32)
    n_fr, n_g1 = block(206, "ffn.proof", ["ffn", "ffn_input.bin", S, E, Hd, work, prefix, "ffn_output.bin"],
                       lambda: orc_check(orc.orc_ffn_block(cu, cf, W[names[6]].h, W[names[7]].h, W[names[8]].h, table, as_fr(f_in), e_out, e_down)))
    f_out = np.fromfile(tmp_path / "ffn_output.bin", dtype=np.int32)
    assert (f_out == fr_to_i64(e_down)).all() and np.abs(f_out).max() > 1000
    run(tmp_path, 206, None, "ffn", "ffn_input.bin", S, E, Hd, work, prefix, "ffn_output_rescaled.bin", extra_env={"ZKLLM_FFN_SAVE_RESCALED": "1"})
    assert (np.fromfile(tmp_path / "ffn_output_rescaled.bin", dtype=np.int32) == fr_to_i64(e_out)).all()
    run(tmp_path, 207, None, "skip-connection", "attn_output.bin", "ffn_output.bin", "layer_output.bin")
    assert (np.fromfile(tmp_path / "layer_output.bin", dtype=np.int32) == x2 + f_out).all()


def test_cross_commitment_side_files_change_no_byte_of_outputs_or_proof(tmp_path):
    """commit-param writes a weight's cross commitments beside its commitment (<commitment>.cross, an addition) and create_weight
    picks them up: the openings of `self-attn linear` then take T, T0, T1 of their first three rounds from them.  16384 generators
    per weight, the smallest set with three such rounds.  The block runs with the side files, without them (every sum over all
    generators), and with the three-round fold tables on top (ZKLLM_OPEN_TABLES=3): the same output files and the same proof
    file, byte for byte, and that proof is the oracle's (field transcript and normalised G1 points)."""
    import ctypes
    orc = load_oracle()
    orc.dll.orc_g1_transcript_size.restype = ctypes.c_long
    S, E, lof = 16, 128, 7
    cu, cf = layercfg.pack(S, E, 2, 256, 1 << 8, 1 << 10, 1 << 7, [1 << 8, 1 << 8, 1 << 8], 1, 0, 1 << 16, [1 << 6, 1 << 8], -512, 1024, 64.0, value_scale=256.0)
    rng = np.random.default_rng(77)
    work = tmp_path / "zkllm-workdir"
    work.mkdir()
    prefix = "layer-0"
    W = {}
    seed = 400
    for name in ("q", "k", "v"):
        full = f"self_attn.{name}_proj.weight"
        w = np.round(rng.normal(0, 0.25, (E, E)) * 256).astype(np.int32)
        pp, ib, cb = work / f"{full}-pp.bin", work / f"{prefix}-{full}-int.bin", work / f"{prefix}-{full}-commitment.bin"
        seed += 1
        run(tmp_path, seed, None, "ppgen", E << lof, pp, config=None)
        w.tofile(ib)
        run(tmp_path, seed, None, "commit-param", pp, ib, cb, E, E, config=None)
        gens, com = g1_file(pp), g1_file(cb)
        assert gens.shape == (E << lof, 36) and com.shape == (1, 36)
        cross = g1_file(str(cb) + ".cross")
        assert cross.shape == (43, 36) and (cross[0] == com[0]).all()          # 1 + 2 + 8 + 32 patterns of one row; pattern 0 is the commitment
        W[name] = OracleWeight(orc, w, E, E, gens, com)
    X = np.round(rng.normal(0, 1, (S, E)) * 256).astype(np.int32)
    X.tofile(tmp_path / "attn_input.bin")
    results = []
    for label, env, hide in (("side files", {}, False), ("no side files", {}, True), ("side files and three-round tables", {"ZKLLM_OPEN_TABLES": "3"}, False)):
        moved = []
        if hide:
            for f in work.glob("*.cross"):
                f.rename(str(f) + ".hidden")
                moved.append(f)
        proof = tmp_path / f"linear_{len(results)}.proof"
        run(tmp_path, 410, proof, "self-attn", "linear", "attn_input.bin", S, E, work, prefix, "unused.bin", extra_env=env)
        for f in moved:
            (f.parent / (f.name + ".hidden")).rename(f)
        results.append((label, open(proof, "rb").read(), [open(tmp_path / f"temp_{n}.bin", "rb").read() for n in "QKV"]))
    for label, pf, outs in results[1:]:
        assert pf == results[0][1], label
        assert outs == results[0][2], label
    eQ, eK, eV = (np.zeros((S * E, 8), np.uint32) for _ in range(3))
    orc.orc_seed(410)
    orc.orc_transcript_clear()
    orc_check(orc.orc_attn_linear_block(cu, cf, W["q"].h, W["k"].h, W["v"].h, as_fr(X), eQ, eK, eV))
    n_fr, n_g1 = check_proof(orc, tmp_path / "linear_0.proof", "side files")
    assert n_g1 == 3 * (3 * 14 + 1)
    Q = np.fromfile(tmp_path / "temp_Q.bin", dtype=np.int32)
    assert (Q == fr_to_i64(eQ)).all()


def test_self_attn_with_heads_from_the_environment_writes_the_output_file(tmp_path):
    """ZKLLM_ATTN_HEADS / ZKLLM_ATTN_HEAD_GROUP (additions): per-head and stacked attention through the executable, against the
    oracle's attention block for the same head count"""
    orc = load_oracle()
    rng = np.random.default_rng(8)
    for group in (0, 2):
        cu, cf = layercfg.tiny(open_weights=False, head_group=group)
        S, E = int(cu[0]), int(cu[1])
        Q, K, V = (np.round(rng.normal(0, 1.0, (S, E)) * 256).astype(np.int32) for _ in range(3))
        for n, t in zip("QKV", (Q, K, V)):
            t.tofile(tmp_path / f"temp_{n}.bin")
        proof = tmp_path / f"heads{group}.proof"
        run(tmp_path, 300 + group, proof, "self-attn", "attn", "unused.bin", S, E, tmp_path, "layer-0", "attn_out.bin",
            extra_env={"ZKLLM_ATTN_HEADS": "2", "ZKLLM_ATTN_HEAD_GROUP": str(group)})
        e = np.zeros((S * E, 8), np.uint32)
        orc.orc_seed(300 + group)
        orc.orc_transcript_clear()
        orc_check(orc.orc_attn_block(cu, cf, 0, as_fr(Q), as_fr(K), as_fr(V), e, None))
        fr, g1 = read_proof(proof)
        exp = orc_transcript(orc)
        assert fr.shape == exp.shape and (fr == exp).all() and g1.shape[0] == 0
        got = np.fromfile(tmp_path / "attn_out.bin", dtype=np.int32)
        assert (got == fr_to_i64(e)).all()
        assert (np.fromfile(tmp_path / "temp_head_out.bin", dtype=np.int32) == got).all()
