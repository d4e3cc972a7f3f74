"""ctypes front-ends of the product libraries for tests, smoke and bench.

Hip     raw C ABI (include/zkllm_hip.h): device buffers are plain integers (addresses)
Prover  class-layer harness (zkp_* in libzkllm_prover.so): tensors are opaque handles
Both fail loudly when the libraries are missing or no GPU is visible; neither has a CPU path.
"""
import ctypes
import importlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
pkg = importlib.import_module("zkllm-ccs2024_amd")

c_void_p, c_size_t, c_int, c_uint, c_u64 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint64


def _np_ptr(a):
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"]
    return c_void_p(a.ctypes.data)


class Hip:
    def __init__(self, device=0):
        self.lib = pkg.load_hip()
        self.check(self.lib.zk_init(c_int(device)))

    def check(self, rc):
        if rc != 0:
            raise RuntimeError(f"zk error {rc}: {self.lib.zk_last_error().decode()}")

    # ---- memory ----
    def malloc(self, nbytes):
        p = c_void_p()
        self.check(self.lib.zk_malloc(ctypes.byref(p), c_size_t(nbytes)))
        return p.value

    def free(self, p):
        self.check(self.lib.zk_free(c_void_p(p)))

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        p = self.malloc(max(arr.nbytes, 1))
        self.check(self.lib.zk_memcpy_h2d(c_void_p(p), _np_ptr(arr), c_size_t(arr.nbytes), None))
        return p

    def download(self, p, shape, dtype):
        out = np.zeros(shape, dtype=dtype)
        self.check(self.lib.zk_memcpy_d2h(_np_ptr(out), c_void_p(p), c_size_t(out.nbytes), None))
        return out

    def sync(self):
        self.check(self.lib.zk_sync(None))

    # ---- generic call: device addresses as ints, numpy arrays as host pointers ----
    def call(self, name, *args):
        fn = getattr(self.lib, name)
        conv = []
        for a in args:
            if isinstance(a, np.ndarray):
                conv.append(_np_ptr(a))
            elif a is None:
                conv.append(c_void_p(None))
            elif isinstance(a, (ctypes._SimpleCData, ctypes._Pointer)) or type(a).__name__ == "CArgObject":
                conv.append(a)
            else:
                conv.append(a)
        self.check(fn(*conv))

    def fr_binary(self, name, a, b):
        n = a.shape[0]
        da, db, do = self.upload(a), self.upload(b), self.malloc(32 * max(n, 1))
        self.call(name, c_void_p(do), c_void_p(da), c_void_p(db), c_size_t(n), None)
        out = self.download(do, (n, 8), np.uint32)
        for p in (da, db, do):
            self.free(p)
        return out

    def fr_unary(self, name, a):
        n = a.shape[0]
        da, do = self.upload(a), self.malloc(32 * max(n, 1))
        self.call(name, c_void_p(do), c_void_p(da), c_size_t(n), None)
        out = self.download(do, (n, 8), np.uint32)
        self.free(da)
        self.free(do)
        return out

    def fr_scalar(self, name, a, s):
        n = a.shape[0]
        da, do = self.upload(a), self.malloc(32 * max(n, 1))
        s = np.ascontiguousarray(s, dtype=np.uint32)
        self.call(name, c_void_p(do), c_void_p(da), s, c_size_t(n), None)
        out = self.download(do, (n, 8), np.uint32)
        self.free(da)
        self.free(do)
        return out


class FrHandle:
    def __init__(self, pv, h):
        if not h:
            raise RuntimeError("prover error: " + pv.lib.zkp_last_error().decode())
        self.pv, self.h = pv, h

    @property
    def size(self):
        return self.pv.lib.zkp_fr_size(c_void_p(self.h))

    @property
    def devptr(self):
        return self.pv.lib.zkp_fr_devptr(c_void_p(self.h))

    def host(self):
        out = np.zeros((self.size, 8), dtype=np.uint32)
        self.pv.check(self.pv.lib.zkp_fr_to_host(c_void_p(self.h), _np_ptr(out)))
        return out

    def __del__(self):
        try:
            self.pv.lib.zkp_fr_free(c_void_p(self.h))
        except Exception:
            pass


class G1Handle:
    def __init__(self, pv, h):
        if not h:
            raise RuntimeError("prover error: " + pv.lib.zkp_last_error().decode())
        self.pv, self.h = pv, h

    @property
    def size(self):
        return self.pv.lib.zkp_g1_size(c_void_p(self.h))

    def host(self):
        out = np.zeros((self.size, 36), dtype=np.uint32)
        self.pv.check(self.pv.lib.zkp_g1_to_host(c_void_p(self.h), _np_ptr(out)))
        return out

    def __del__(self):
        try:
            self.pv.lib.zkp_g1_free(c_void_p(self.h))
        except Exception:
            pass


class Prover:
    def __init__(self, device=0):
        self.lib = pkg.load_prover()
        L = self.lib
        for name in ("zkp_fr_from_i32", "zkp_fr_from_i64", "zkp_fr_from_fr", "zkp_fr_from_f32", "zkp_fr_from_f64", "zkp_fr_from_file",
                     "zkp_fr_devptr", "zkp_fr_binop", "zkp_fr_scalarop", "zkp_fr_partial_me", "zkp_fr_partial_me_window",
                     "zkp_fr_pad", "zkp_fr_split", "zkp_fr_transpose", "zkp_fr_matmul", "zkp_fr_matmul_stack", "zkp_fr_transpose_stack", "zkp_fr_matmul_stack_prod", "zkp_fr_partial_me_prod", "zkp_fr_swap_axes",
                     "zkp_g1_from_host", "zkp_g1_from_file", "zkp_g1_devptr", "zkp_commitment_random", "zkp_g1_binop", "zkp_g1_pointop", "zkp_g1_affineop",
                     "zkp_g1_scalar_mul", "zkp_g1_rowwise_sum", "zkp_commit_int", "zkp_commit",
                     "zkp_rescale", "zkp_rescale_prove", "zkp_relu", "zkp_attn", "zkp_zkfc_stacked", "zkp_range_prep", "zkp_batch_inv", "zkp_softmax",
                     "zkp_layer_create", "zkp_layer_create_random", "zkp_layer_run", "zkp_fc_forward_over_view"):
            getattr(L, name).restype = c_void_p
        L.zkp_rescale_ints_prove.restype = c_void_p
        L.zkp_transcript_size.restype = ctypes.c_long
        L.zkp_fr_size.restype = c_uint
        L.zkp_g1_size.restype = c_uint
        self.check(L.zkp_init(c_int(device)))

    def check(self, rc):
        if rc != 0:
            raise RuntimeError("prover error: " + self.lib.zkp_last_error().decode())

    def H(self, h):
        return FrHandle(self, h)

    # ---- tensors ----
    def from_i32(self, a):
        a = np.ascontiguousarray(a, dtype=np.int32)
        return self.H(self.lib.zkp_fr_from_i32(_np_ptr(a), c_uint(a.size)))

    def from_i64(self, a):
        a = np.ascontiguousarray(a, dtype=np.int64)
        return self.H(self.lib.zkp_fr_from_i64(_np_ptr(a), c_uint(a.size)))

    def from_fr(self, a):
        a = np.ascontiguousarray(a, dtype=np.uint32).reshape(-1, 8)
        return self.H(self.lib.zkp_fr_from_fr(_np_ptr(a), c_uint(a.shape[0])))

    def from_f32(self, a, sf):
        a = np.ascontiguousarray(a, dtype=np.float32)
        return self.H(self.lib.zkp_fr_from_f32(_np_ptr(a), c_uint(a.size), c_u64(sf)))

    def from_f64(self, a, sf):
        a = np.ascontiguousarray(a, dtype=np.float64)
        return self.H(self.lib.zkp_fr_from_f64(_np_ptr(a), c_uint(a.size), c_u64(sf)))

    def from_file(self, path, kind):
        """kind 0: raw field elements (FrTensor(filename)), 1: int32 (from_int_bin), 2: int64 (from_long_bin)"""
        return self.H(self.lib.zkp_fr_from_file(str(path).encode(), c_int(kind)))

    def save(self, t, path, kind):
        """kind 0: save, 1: save_int, 2: save_long"""
        self.check(self.lib.zkp_fr_save(c_void_p(t.h), str(path).encode(), c_int(kind)))

    def binop(self, op, a, b):
        return self.H(self.lib.zkp_fr_binop(c_int(op), c_void_p(a.h), c_void_p(b.h)))

    def scalarop(self, op, a, s=None):
        s = np.zeros(8, np.uint32) if s is None else np.ascontiguousarray(s, dtype=np.uint32)
        return self.H(self.lib.zkp_fr_scalarop(c_int(op), c_void_p(a.h), _np_ptr(s)))

    def sum(self, a):
        out = np.zeros(8, np.uint32)
        self.check(self.lib.zkp_fr_sum(c_void_p(a.h), _np_ptr(out)))
        return out

    def me(self, a, u):
        u = np.ascontiguousarray(u, dtype=np.uint32).reshape(-1, 8)
        out = np.zeros(8, np.uint32)
        self.check(self.lib.zkp_fr_me(c_void_p(a.h), _np_ptr(u), c_int(u.shape[0]), _np_ptr(out)))
        return out

    def partial_me(self, a, u, cur_dim, window):
        u = np.ascontiguousarray(u, dtype=np.uint32).reshape(-1, 8)
        return self.H(self.lib.zkp_fr_partial_me(c_void_p(a.h), _np_ptr(u), c_int(u.shape[0]), c_uint(cur_dim), c_uint(window)))

    def partial_me_window(self, a, u, window):
        u = np.ascontiguousarray(u, dtype=np.uint32).reshape(-1, 8)
        return self.H(self.lib.zkp_fr_partial_me_window(c_void_p(a.h), _np_ptr(u), c_int(u.shape[0]), c_uint(window)))

    def multi_dim_me(self, a, us, shape):
        cat = np.ascontiguousarray(np.concatenate([np.asarray(u, dtype=np.uint32).reshape(-1, 8) for u in us]) if us else np.zeros((0, 8), np.uint32))
        lens = np.array([np.asarray(u).reshape(-1, 8).shape[0] for u in us], dtype=np.uint32)
        shp = np.array(shape, dtype=np.uint32)
        out = np.zeros(8, np.uint32)
        self.check(self.lib.zkp_fr_multi_dim_me(c_void_p(a.h), _np_ptr(cat), _np_ptr(lens), _np_ptr(shp), c_int(len(shape)), _np_ptr(out)))
        return out

    def pad(self, a, shape, pad_val=None):
        pv = np.zeros(8, np.uint32) if pad_val is None else np.ascontiguousarray(pad_val, dtype=np.uint32)
        shp = np.array(shape, dtype=np.uint32)
        return self.H(self.lib.zkp_fr_pad(c_void_p(a.h), _np_ptr(shp), c_int(len(shape)), _np_ptr(pv)))

    def transpose(self, a, M, N):
        return self.H(self.lib.zkp_fr_transpose(c_void_p(a.h), c_uint(M), c_uint(N)))

    def matmul(self, a, b, M, N, P):
        return self.H(self.lib.zkp_fr_matmul(c_void_p(a.h), c_void_p(b.h), c_uint(M), c_uint(N), c_uint(P)))

    def keep_as_matmul_rhs(self, a):
        self.check(self.lib.zkp_fr_keep_as_matmul_rhs(c_void_p(a.h)))

    def keep_for_folds(self, a):
        self.check(self.lib.zkp_fr_keep_for_folds(c_void_p(a.h)))

    def folds_from_ints(self, a):
        return int(self.lib.zkp_fr_folds_from_ints(c_void_p(a.h)))

    def add_inplace(self, a, b):
        self.check(self.lib.zkp_fr_add_inplace(c_void_p(a.h), c_void_p(b.h)))

    def fc_forward_over_view(self, w, x, in_dim, out_dim):
        return self.H(self.lib.zkp_fc_forward_over_view(c_void_p(w.h), c_void_p(x.h), c_uint(in_dim), c_uint(out_dim)))

    def matmul_stack(self, a, b, num, M, N, P):
        return self.H(self.lib.zkp_fr_matmul_stack(c_void_p(a.h), c_void_p(b.h), c_uint(num), c_uint(M), c_uint(N), c_uint(P)))

    def swap_axes(self, a, A, B, C):
        return self.H(self.lib.zkp_fr_swap_axes(c_void_p(a.h), c_uint(A), c_uint(B), c_uint(C)))

    def matmul_stack_prod(self, a, b, y, num, M, N, P):
        return self.H(self.lib.zkp_fr_matmul_stack_prod(c_void_p(a.h), c_void_p(b.h), c_void_p(y.h), c_uint(num), c_uint(M), c_uint(N), c_uint(P)))

    def partial_me_prod(self, a, b, u, cur_dim, window):
        return self.H(self.lib.zkp_fr_partial_me_prod(c_void_p(a.h), c_void_p(b.h), _np_ptr(u), c_int(u.shape[0]), c_uint(cur_dim), c_uint(window)))

    def transpose_stack(self, a, num, M, N):
        return self.H(self.lib.zkp_fr_transpose_stack(c_void_p(a.h), c_uint(num), c_uint(M), c_uint(N)))

    # ---- G1 ----
    def G(self, h):
        return G1Handle(self, h)

    def g1_from_host(self, pts):
        pts = np.ascontiguousarray(pts, dtype=np.uint32).reshape(-1, 36)
        return self.G(self.lib.zkp_g1_from_host(_np_ptr(pts), c_uint(pts.shape[0])))

    def commitment_random(self, size):
        return self.G(self.lib.zkp_commitment_random(c_uint(size)))

    def g1_binop(self, op, a, b=None):
        return self.G(self.lib.zkp_g1_binop(c_int(op), c_void_p(a.h), c_void_p(b.h if b is not None else a.h)))

    def g1_pointop(self, op, a, p):
        p = np.ascontiguousarray(p, dtype=np.uint32).reshape(36)
        return self.G(self.lib.zkp_g1_pointop(c_int(op), c_void_p(a.h), _np_ptr(p)))

    def g1_affineop(self, op, a, aff, path=None):
        aff = np.ascontiguousarray(aff, dtype=np.uint32).reshape(-1, 24)
        return self.G(self.lib.zkp_g1_affineop(c_int(op), c_void_p(a.h), _np_ptr(aff), c_uint(aff.shape[0]),
                                               ctypes.c_char_p(path.encode() if path else None)))

    def g1_scalar_mul(self, g, s):
        return self.G(self.lib.zkp_g1_scalar_mul(c_void_p(g.h), c_void_p(s.h)))

    def g1_sum(self, a):
        out = np.zeros(36, np.uint32)
        self.check(self.lib.zkp_g1_sum(c_void_p(a.h), _np_ptr(out)))
        return out

    def g1_rowwise_sum(self, a, nrow, ncol):
        return self.G(self.lib.zkp_g1_rowwise_sum(c_void_p(a.h), c_uint(nrow), c_uint(ncol)))

    def g1_me(self, a, u):
        u = np.ascontiguousarray(u, dtype=np.uint32).reshape(-1, 8)
        out = np.zeros(36, np.uint32)
        self.check(self.lib.zkp_g1_me(c_void_p(a.h), _np_ptr(u), c_int(u.shape[0]), _np_ptr(out)))
        return out

    def commit_int(self, gens, t):
        return self.G(self.lib.zkp_commit_int(c_void_p(gens.h), c_void_p(t.h)))

    def commit(self, gens, t):
        return self.G(self.lib.zkp_commit(c_void_p(gens.h), c_void_p(t.h)))

    def open(self, gens, t, com, u):
        u = np.ascontiguousarray(u, dtype=np.uint32).reshape(-1, 8)
        k = u.shape[0]
        proof = np.zeros((3 * k + 1, 36), np.uint32)
        npf = c_int(0)
        val = np.zeros(8, np.uint32)
        self.check(self.lib.zkp_open(c_void_p(gens.h), c_void_p(t.h), c_void_p(com.h), _np_ptr(u), c_int(k), _np_ptr(proof), ctypes.byref(npf), _np_ptr(val)))
        return val, proof[:npf.value]

    # ---- lookup / rescaling / softmax ----
    def rescale(self, X, sf):
        rem = c_void_p()
        out = self.H(self.lib.zkp_rescale(c_void_p(X.h), c_uint(sf), ctypes.byref(rem)))
        return out, self.H(rem.value)

    def relu(self, X, sf):
        parts = (c_void_p * 4)()
        out = self.H(self.lib.zkp_relu(c_void_p(X.h), c_uint(sf), parts))
        return out, [self.H(p) for p in parts]

    def rescale_ints_prove(self, X, sf):
        return self.H(self.lib.zkp_rescale_ints_prove(c_void_p(X.h), c_uint(sf)))

    def rescale_prove(self, X, sf):
        return self.H(self.lib.zkp_rescale_prove(c_void_p(X.h), c_uint(sf)))

    def range_prep(self, vals, low, length):
        return self.H(self.lib.zkp_range_prep(c_void_p(vals.h), c_int(low), c_uint(length)))

    def batch_inv(self, a, beta):
        beta = np.ascontiguousarray(beta, dtype=np.uint32)
        return self.H(self.lib.zkp_batch_inv(c_void_p(a.h), _np_ptr(beta)))

    def range_prove(self, S, low, length, alpha, beta, u, v):
        fin = np.zeros(8, np.uint32)
        args = [np.ascontiguousarray(x, dtype=np.uint32) for x in (alpha, beta, u, v)]
        self.check(self.lib.zkp_range_prove(c_void_p(S.h), c_int(low), c_uint(length), *[_np_ptr(a) for a in args], _np_ptr(fin)))
        return fin

    def mapping(self, S_in, low, length, mvals, r=None, alpha=None, beta=None, u=None, v=None):
        y, m = c_void_p(), c_void_p()
        prove = r is not None
        fin = np.zeros(8, np.uint32)
        z = np.zeros(8, np.uint32)
        args = [np.ascontiguousarray(x if x is not None else z, dtype=np.uint32) for x in (r, alpha, beta, u, v)]
        self.check(self.lib.zkp_mapping(c_void_p(S_in.h), c_int(low), c_uint(length), c_void_p(mvals.h), *[_np_ptr(a) for a in args],
                                        ctypes.byref(y), ctypes.byref(m), _np_ptr(fin) if prove else None))
        return self.H(y.value), self.H(m.value), fin

    def multi_hadamard(self, claim, Xs, u, v):
        u = np.ascontiguousarray(u, dtype=np.uint32).reshape(-1, 8)
        v = np.ascontiguousarray(v, dtype=np.uint32).reshape(-1, 8)
        k = u.shape[0]
        arr = (c_void_p * len(Xs))(*[x.h for x in Xs])
        proof = np.zeros((k * (len(Xs) + 1), 8), np.uint32)
        fin = np.zeros(8, np.uint32)
        claim = np.ascontiguousarray(claim, dtype=np.uint32)
        self.check(self.lib.zkp_multi_hadamard(_np_ptr(claim), arr, c_int(len(Xs)), _np_ptr(u), _np_ptr(v), c_int(k), _np_ptr(proof), _np_ptr(fin)))
        return proof, fin

    def hadamard_product_sumcheck(self, a, b, u, v):
        u = np.ascontiguousarray(u, dtype=np.uint32).reshape(-1, 8)
        v = np.ascontiguousarray(v, dtype=np.uint32).reshape(-1, 8)
        k = u.shape[0]
        proof = np.zeros((3 * k + 2, 8), np.uint32)
        self.check(self.lib.zkp_hadamard_product_sumcheck(c_void_p(a.h), c_void_p(b.h), _np_ptr(u), _np_ptr(v), c_int(k), _np_ptr(proof)))
        return proof

    def inner_product_sumcheck(self, a, b, u):
        u = np.ascontiguousarray(u, dtype=np.uint32).reshape(-1, 8)
        k = u.shape[0]
        proof = np.zeros((3 * k + 2, 8), np.uint32)
        self.check(self.lib.zkp_inner_product_sumcheck(c_void_p(a.h), c_void_p(b.h), _np_ptr(u), c_int(k), _np_ptr(proof)))
        return proof

    def binary_sumcheck(self, a, u, v):
        u = np.ascontiguousarray(u, dtype=np.uint32).reshape(-1, 8)
        v = np.ascontiguousarray(v, dtype=np.uint32).reshape(-1, 8)
        k = u.shape[0]
        proof = np.zeros((3 * k + 1, 8), np.uint32)
        self.check(self.lib.zkp_binary_sumcheck(c_void_p(a.h), _np_ptr(u), _np_ptr(v), c_int(k), _np_ptr(proof)))
        return proof

    def split(self, t, window):
        odd = c_void_p()
        even = self.H(self.lib.zkp_fr_split(c_void_p(t.h), c_uint(window), ctypes.byref(odd)))
        return even, self.H(odd.value)

    def softmax(self, X, m, n, d, bs, L, M, sf_in, thetas, prove):
        bs = np.ascontiguousarray(bs, dtype=np.uint32)
        thetas = np.ascontiguousarray(thetas, dtype=np.float64)
        shift = c_void_p()
        y = self.H(self.lib.zkp_softmax(c_void_p(X.h), c_uint(m), c_uint(n), c_uint(d), _np_ptr(bs), c_int(len(bs)), c_uint(L), c_uint(M), c_u64(sf_in),
                                        _np_ptr(thetas), c_int(len(thetas)), ctypes.byref(shift), c_int(1 if prove else 0)))
        return y, self.H(shift.value)

    def attn(self, Q, K, V, num, m, n, d, stacked, bs, L, M, sf_Q, sf_K, thetas):
        bs = np.ascontiguousarray(bs, dtype=np.uint32)
        th = np.ascontiguousarray(thetas, dtype=np.float64)
        fin = np.zeros(8, np.uint32)
        out = self.H(self.lib.zkp_attn(c_void_p(Q.h), c_void_p(K.h), c_void_p(V.h), c_uint(num), c_uint(m), c_uint(n), c_uint(d), c_int(int(stacked)),
                                       _np_ptr(bs), c_int(len(bs)), c_uint(L), c_uint(M), ctypes.c_uint64(sf_Q), ctypes.c_uint64(sf_K),
                                       th.ctypes.data_as(c_void_p), c_int(len(th)), _np_ptr(fin)))
        return out, fin

    def zkfc_stacked(self, X, W, b, num, batch, n_in, n_out):
        return self.H(self.lib.zkp_zkfc_stacked(c_void_p(X.h), c_void_p(W.h), c_void_p(b.h) if b is not None else None, c_uint(num), c_uint(batch),
                                                c_uint(n_in), c_uint(n_out)))

    def zkip_stacked(self, claim, A, B, N, D, uN, vN, uD):
        uN, vN, uD = (np.ascontiguousarray(x, dtype=np.uint32).reshape(-1, 8) for x in (uN, vN, uD))
        kN, kD = uN.shape[0], uD.shape[0]
        proof = np.zeros((kN + kD, 3, 8), np.uint32)
        fin = np.zeros(8, np.uint32)
        claim = np.ascontiguousarray(claim, dtype=np.uint32)
        self.check(self.lib.zkp_zkip_stacked(_np_ptr(claim), c_void_p(A.h), c_void_p(B.h), c_uint(N), c_uint(D), _np_ptr(uN), _np_ptr(vN), c_int(kN),
                                             _np_ptr(uD), c_int(kD), _np_ptr(proof), _np_ptr(fin)))
        return proof, fin

    # ---- decoder layer ----
    def layer_create(self, cu, cf, weights, log_off_factor):
        ws = [np.ascontiguousarray(w, dtype=np.int32) for w in weights]
        h = self.lib.zkp_layer_create(_np_ptr(cu), _np_ptr(cf), *[_np_ptr(w) for w in ws], c_uint(log_off_factor))
        if not h:
            raise RuntimeError("prover error: " + self.lib.zkp_last_error().decode())
        return h

    def layer_create_random(self, cu, cf, seed, log_off_factor):
        h = self.lib.zkp_layer_create_random(_np_ptr(cu), _np_ptr(cf), c_uint(seed), c_uint(log_off_factor))
        if not h:
            raise RuntimeError("prover error: " + self.lib.zkp_last_error().decode())
        return h

    def layer_run(self, layer, X):
        times = np.zeros(8, np.float64)
        out = self.H(self.lib.zkp_layer_run(c_void_p(layer), c_void_p(X.h), _np_ptr(times)))
        return out, times

    def layer_set(self, layer, head_group=None, open_weights=None):
        if head_group is not None:
            self.lib.zkp_layer_set_head_group(c_void_p(layer), c_uint(head_group))
        if open_weights is not None:
            self.lib.zkp_layer_set_open_weights(c_void_p(layer), c_int(1 if open_weights else 0))

    def layer_free(self, layer):
        self.lib.zkp_layer_free(c_void_p(layer))

    # ---- transcript / challenges ----
    def seed(self, s):
        self.lib.zkp_seed(c_uint(s))

    def transcript_begin(self):
        self.lib.zkp_transcript_begin()

    def transcript(self):
        n = self.lib.zkp_transcript_size()
        out = np.zeros((n, 8), dtype=np.uint32)
        if n:
            self.lib.zkp_transcript_get(_np_ptr(out))
        return out

    def transcript_g1(self):
        self.lib.zkp_transcript_g1_size.restype = ctypes.c_long
        n = self.lib.zkp_transcript_g1_size()
        out = np.zeros((n, 36), dtype=np.uint32)
        if n:
            self.lib.zkp_transcript_g1_get(_np_ptr(out))
        return out

    def sync(self):
        self.check(self.lib.zkp_sync())

    # ---- protocols ----
    def zkip(self, claim, a, b, u):
        u = np.ascontiguousarray(u, dtype=np.uint32).reshape(-1, 8)
        k = u.shape[0]
        proof = np.zeros((k, 3, 8), np.uint32)
        fin = np.zeros(8, np.uint32)
        claim = np.ascontiguousarray(claim, dtype=np.uint32)
        self.check(self.lib.zkp_zkip(_np_ptr(claim), c_void_p(a.h), c_void_p(b.h), _np_ptr(u), c_int(k), _np_ptr(proof), _np_ptr(fin)))
        return proof, fin

    def zkfc_prove(self, X, W, Y, in_dim, out_dim):
        cw = np.zeros(8, np.uint32)
        self.check(self.lib.zkp_zkfc_prove(c_void_p(X.h), c_void_p(W.h), c_void_p(Y.h), c_uint(in_dim), c_uint(out_dim), _np_ptr(cw)))
        return cw

    def zkfc_scenario(self, X, W, seed, matmul_mode=0):
        """forward + prove on int32 inputs; returns (Y as Fr limbs, transcript)"""
        B, I = X.shape
        O = W.shape[1]
        self.lib.zkp_set_matmul_mode(c_int(matmul_mode))
        hX, hW = self.from_i32(X), self.from_i32(W)
        hY = self.matmul(hX, hW, B, I, O)
        self.seed(seed)
        self.transcript_begin()
        self.zkfc_prove(hX, hW, hY, I, O)
        self.lib.zkp_transcript_end()
        return hY.host(), self.transcript()
