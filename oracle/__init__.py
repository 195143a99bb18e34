"""ctypes front end of the CPU checker (oracle/tg_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of bench.py.  The shipped package never imports it.
"""
import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB = None
_REF = None
_REF_IO = None

f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")


class OrcModel(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("depth", "context", "batch", "d_model", "heads", "vocab", "ffn")] + [
        ("ln_eps", C.c_float), ("emulate", C.c_int)]


def build():
    """Compile liborc.so (and oracle/_ref when the reference tree is mounted)."""
    subprocess.run(["make", "-C", str(_HERE), "-s", "all"], check=True)


def lib():
    global _LIB
    if _LIB is None:
        path = _HERE / "liborc.so"
        if not path.exists():
            build()
        _LIB = C.CDLL(str(path))
        _LIB.orc_hash_u64.restype = C.c_uint64
        _LIB.orc_hash_u64.argtypes = [C.c_uint64]
        _LIB.orc_bf16_round.restype = C.c_float
        _LIB.orc_bf16_round.argtypes = [C.c_float]
        _LIB.orc_bf16_trunc.restype = C.c_float
        _LIB.orc_bf16_trunc.argtypes = [C.c_float]
        _LIB.orc_clip_scale.restype = C.c_float
        _LIB.orc_parameter_count.restype = C.c_int64
    return _LIB


def ref_host():
    """The reference's own onecycle_point/hash_u64, or None when oracle/_ref was never built."""
    global _REF
    if _REF is None:
        path = _HERE / "_ref" / "libtgref_host.so"
        if not path.exists():
            return None
        _REF = C.CDLL(str(path))
        _REF.tgref_hash_u64.restype = C.c_uint64
        _REF.tgref_hash_u64.argtypes = [C.c_uint64]
    return _REF


def ref_io():
    """The reference's own checkpoint / loss-summary / event-file code behind C linkage (oracle/ref_host_io_shim.cpp),
    or None when oracle/_ref was never built."""
    global _REF_IO
    if _REF_IO is None:
        path = _HERE / "_ref" / "libtgref_io.so"
        if not path.exists():
            return None
        _REF_IO = C.CDLL(str(path))
        _REF_IO.tgref_io_error.restype = C.c_char_p
        _REF_IO.tgref_events_open.restype = C.c_void_p
        _REF_IO.tgref_events_open.argtypes = [C.c_char_p]
        _REF_IO.tgref_events_scalar.argtypes = [C.c_void_p, C.c_char_p, C.c_double, C.c_int64]
        _REF_IO.tgref_events_text.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_int64]
        _REF_IO.tgref_events_close.argtypes = [C.c_void_p]
    return _REF_IO


def _f(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def hash_u64(x):
    return int(lib().orc_hash_u64(C.c_uint64(x & (2**64 - 1))))


def bf16_round(a):
    a = _f(a).copy()
    lib().orc_bf16_round_array(_p(a), C.c_int64(a.size))
    return a


def bf16_trunc(a):
    a = _f(a).copy()
    lib().orc_bf16_trunc_array(_p(a), C.c_int64(a.size))
    return a


def split_hilo(w):
    w = _f(w)
    hi, lo = np.empty(w.size, np.uint16), np.empty(w.size, np.uint16)
    lib().orc_split_hilo(_p(w), _p(hi), _p(lo), C.c_int64(w.size))
    return hi, lo


def join_hilo(hi, lo):
    hi, lo = np.ascontiguousarray(hi, np.uint16), np.ascontiguousarray(lo, np.uint16)
    w = np.empty(hi.size, np.float32)
    lib().orc_join_hilo(_p(hi), _p(lo), _p(w), C.c_int64(hi.size))
    return w


def fill_normal(n, seed, scale=1.0):
    out = np.empty(n, np.float32)
    lib().orc_fill_normal(_p(out), C.c_int64(n), C.c_uint64(seed), C.c_float(scale))
    return out


def fill_uniform_bytes(n, seed):
    out = np.empty(n, np.uint8)
    lib().orc_fill_uniform_bytes(_p(out), C.c_int64(n), C.c_uint64(seed))
    return out


def fill_zipf_bytes(n, seed, s=1.1):
    out = np.empty(n, np.uint8)
    lib().orc_fill_zipf_bytes(_p(out), C.c_int64(n), C.c_uint64(seed), C.c_double(s))
    return out


def gemm_fwd(x, w, residual=None, emulate=False):
    x, w = _f(x), _f(w)
    (M, K), N = x.shape, w.shape[0]
    assert w.shape[1] == K
    y = np.empty((M, N), np.float32)
    r = _f(residual) if residual is not None else None
    lib().orc_gemm_fwd(M, N, K, _p(x), K, _p(w), K, _p(y), N, _p(r), N, int(emulate))
    return y


def gemm_dgrad(dy, w, emulate=False):
    dy, w = _f(dy), _f(w)
    (M, N), K = dy.shape, w.shape[1]
    assert w.shape[0] == N
    dx = np.empty((M, K), np.float32)
    lib().orc_gemm_dgrad(M, N, K, _p(dy), N, _p(w), K, _p(dx), K, int(emulate))
    return dx


def gemm_wgrad(dy, x, into=None):
    dy, x = _f(dy), _f(x)
    (M, N), K = dy.shape, x.shape[1]
    assert x.shape[0] == M
    dw = np.zeros((N, K), np.float32) if into is None else _f(into).copy()
    lib().orc_gemm_wgrad(M, N, K, _p(dy), N, _p(x), K, _p(dw), K, int(into is not None))
    return dw


def attn_fwd(qkv, B, H, T, hd, scale, emulate=False):
    qkv = _f(qkv)
    d = H * hd
    assert qkv.shape == (B * T, 3 * d)
    out = np.empty((B * T, d), np.float32)
    lse = np.empty((B, H, T), np.float32)
    lib().orc_attn_fwd(B, H, T, hd, _p(qkv), 3 * d, _p(out), d, _p(lse), C.c_float(scale), int(emulate))
    return out, lse


def attn_bwd(qkv, out, lse, dout, B, H, T, hd, scale, emulate=False):
    qkv, out, lse, dout = _f(qkv), _f(out), _f(lse), _f(dout)
    d = H * hd
    dqkv = np.empty((B * T, 3 * d), np.float32)
    lib().orc_attn_bwd(B, H, T, hd, _p(qkv), 3 * d, _p(out), d, _p(lse), _p(dout), d, _p(dqkv), 3 * d,
                       C.c_float(scale), int(emulate))
    return dqkv


def layernorm_fwd(x, gamma, beta, eps=1e-5, emulate=False):
    x, gamma, beta = _f(x), _f(gamma), _f(beta)
    y = np.empty_like(x)
    lib().orc_layernorm_fwd(x.shape[0], x.shape[1], _p(x), _p(gamma), _p(beta), _p(y), C.c_float(eps),
                            int(emulate))
    return y


def layernorm_bwd(x, dy, gamma, eps=1e-5, dx_in=None, emulate=False):
    x, dy, gamma = _f(x), _f(dy), _f(gamma)
    dx = np.zeros_like(x) if dx_in is None else _f(dx_in).copy()
    dg, db = np.zeros(x.shape[1], np.float32), np.zeros(x.shape[1], np.float32)
    lib().orc_layernorm_bwd(x.shape[0], x.shape[1], _p(x), _p(dy), _p(gamma), _p(dx), _p(dg), _p(db),
                            C.c_float(eps), int(dx_in is not None), int(emulate))
    return dx, dg, db


def gelu_fwd(u, emulate=False):
    u = _f(u)
    a = np.empty_like(u)
    lib().orc_gelu_fwd(C.c_int64(u.size), _p(u), _p(a), int(emulate))
    return a


def gelu_bwd(u, da, emulate=False):
    u, da = _f(u), _f(da)
    du = np.empty_like(u)
    lib().orc_gelu_bwd(C.c_int64(u.size), _p(u), _p(da), _p(du), int(emulate))
    return du


def cross_entropy(logits, y, inv_count=None, emulate=False):
    logits, y = _f(logits), np.ascontiguousarray(y, np.uint8)
    M, V = logits.shape
    loss, dl = np.empty(M, np.float32), np.empty((M, V), np.float32)
    inv = 1.0 / M if inv_count is None else inv_count
    lib().orc_cross_entropy(M, V, _p(logits), _p(y), _p(loss), _p(dl), C.c_float(inv), int(emulate))
    return loss, dl


def adamw(w, m, v, g, decay, lr, beta1, beta2, eps, weight_decay, clip_scale, step):
    w, m, v, g = _f(w).copy(), _f(m).copy(), _f(v).copy(), _f(g)
    decay = np.ascontiguousarray(decay, np.uint8)
    lib().orc_adamw(C.c_int64(w.size), _p(w), _p(m), _p(v), _p(g), _p(decay), C.c_float(lr),
                    C.c_float(beta1), C.c_float(beta2), C.c_float(eps), C.c_float(weight_decay),
                    C.c_float(clip_scale), C.c_uint64(step))
    return w, m, v


def clip_scale(g, clip):
    g = _f(g)
    return float(lib().orc_clip_scale(C.c_int64(g.size), _p(g), C.c_float(clip)))


def onecycle_point(total, step, warmup=0.30, initial=0.04, final=0.000004, low=0.85, high=0.95, use_ref=False):
    mult, mom = C.c_float(), C.c_float()
    fn = ref_host().tgref_onecycle_point if use_ref else lib().orc_onecycle_point
    rc = fn(total, C.c_double(warmup), C.c_double(initial), C.c_double(final), C.c_double(low),
            C.c_double(high), step, C.byref(mult), C.byref(mom))
    if rc:
        raise ValueError("Invalid OneCycle schedule or step")
    return mult.value, mom.value


def sample_batch(data, seed, step, batch, context):
    data = np.ascontiguousarray(data, np.uint8)
    x, y = np.empty((batch, context), np.uint8), np.empty((batch, context), np.uint8)
    lib().orc_sample_batch(_p(data), C.c_int64(data.size), C.c_uint64(seed), C.c_uint64(step), batch,
                           context, _p(x), _p(y))
    return x, y


def model(depth, context, batch, d_model, heads, vocab=256, ffn=None, ln_eps=1e-5, emulate=False):
    return OrcModel(depth, context, batch, d_model, heads, vocab, ffn or 4 * d_model, ln_eps, int(emulate))


def parameter_count(cfg):
    return int(lib().orc_parameter_count(C.byref(cfg)))


class Layout:
    """Offsets of the flat parameter vector, by name."""

    def __init__(self, cfg):
        d, F, V, T = cfg.d_model, cfg.ffn, cfg.vocab, cfg.context
        self.entries = []
        n = 0

        def take(name, shape):
            nonlocal n
            size = int(np.prod(shape))
            self.entries.append((name, n, shape))
            n += size

        take("embedding", (V, d))
        take("positions", (T, d))
        for l in range(cfg.depth):
            for name, shape in [("ln1_g", (d,)), ("ln1_b", (d,)), ("qkv", (3 * d, d)), ("attn_out", (d, d)),
                                ("ln2_g", (d,)), ("ln2_b", (d,)), ("mlp_up", (F, d)), ("mlp_down", (d, F))]:
                take(f"{l}.{name}", shape)
        take("lnf_g", (d,))
        take("lnf_b", (d,))
        take("head", (V, d))
        self.count = n


def decay_mask(cfg):
    mask = np.empty(parameter_count(cfg), np.uint8)
    lib().orc_decay_mask(C.byref(cfg), _p(mask))
    return mask


def init_weights(cfg, seed=3407, scale=0.02):
    w = np.empty(parameter_count(cfg), np.float32)
    lib().orc_init_weights(C.byref(cfg), C.c_uint64(seed), C.c_float(scale), _p(w))
    return w


def model_batch(cfg, params, x, y, backward=True):
    params = _f(params)
    x, y = np.ascontiguousarray(x, np.uint8), np.ascontiguousarray(y, np.uint8)
    M = cfg.batch * cfg.context
    assert x.size == M and y.size == M and params.size == parameter_count(cfg)
    logits = np.empty((cfg.batch, cfg.context, cfg.vocab), np.float32)
    grad = np.empty(params.size, np.float32) if backward else None
    loss = np.empty((cfg.batch, cfg.context), np.float32)
    rc = lib().orc_model_batch(C.byref(cfg), _p(params), _p(x), _p(y), _p(logits), _p(grad), _p(loss))
    assert rc == 0
    return logits, grad, loss


def train(cfg, params, m, v, data, seed, first_step, steps, lr, beta1, beta2, eps, weight_decay, clip,
          multipliers=None, momenta=None):
    params, m, v = _f(params).copy(), _f(m).copy(), _f(v).copy()
    data = np.ascontiguousarray(data, np.uint8)
    losses = np.empty((steps, cfg.context), np.float32)
    mu = _f(multipliers) if multipliers is not None else None
    mo = _f(momenta) if momenta is not None else None
    rc = lib().orc_train(C.byref(cfg), _p(params), _p(m), _p(v), _p(data), C.c_int64(data.size),
                         C.c_uint64(seed), C.c_uint64(first_step), steps, C.c_float(lr), C.c_float(beta1),
                         C.c_float(beta2), C.c_float(eps), C.c_float(weight_decay), C.c_float(clip),
                         _p(mu), _p(mo), _p(losses))
    assert rc == 0
    return params, m, v, losses


def threads():
    return int(lib().orc_threads())
