"""ctypes interface to libturbogpt.so.

Mirrors the reference's tests/bridge.py (Config / OneCycle / StepRates / Native over the tg_* ABI,
bridge.py:7-81) and adds the kernel-level tgk_* entry points.  There is no fallback: if the HIP
library is missing or a symbol is absent, loading raises.
"""
import ctypes as C
import os
from pathlib import Path

_HERE = Path(__file__).resolve().parent
_LIB = None

vp, i32, i64, f32, sz = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_size_t

# name -> (restype, argtypes); every symbol include/tgk_kernels.h declares
KERNEL_ABI = {
    "tgk_error": (C.c_char_p, []),
    "tgk_gemm_fwd": (i32, [vp, i32, i32, i32, vp, i32, vp, i32, vp, i32, vp, i32, vp, i32]),
    "tgk_gemm_fwd_t": (i32, [vp, i32, i32, i32, vp, i32, vp, i32, vp, i32, vp, i32, vp, i32]),
    "tgk_transpose_batch": (i32, [vp, vp, vp, vp, i32, i32]),
    "tgk_gemm_dgrad": (i32, [vp, i32, i32, i32, vp, i32, vp, i32, vp, i32, vp, i32]),
    "tgk_gemm_dgrad_t": (i32, [vp, i32, i32, i32, vp, i32, vp, i32, vp, i32, vp, i32]),
    "tgk_gemm_wgrad": (i32, [vp, i32, i32, i32, vp, i32, vp, i32, vp, i32, i32, vp, sz]),
    "tgk_gemm_wgrad_workspace": (sz, [i32, i32, i32]),
    "tgk_gemm_wgrad_batch": (i32, [vp, i32, i32, vp, i32, vp, sz]),
    "tgk_gemm_wgrad_batch_workspace": (sz, [i32, i32, vp]),
    "tgk_gemm_wgrad_list_table_bytes": (sz, [i32, i32, vp]),
    "tgk_gemm_wgrad_list_workspace": (sz, [i32, i32, vp]),
    "tgk_gemm_wgrad_list_prepare": (i32, [i32, i32, vp, vp, sz]),
    "tgk_gemm_wgrad_list": (i32, [vp, i32, i32, vp, vp, i32, vp, sz, vp]),
    "tgk_gemm_wgrad_list_sumsq_count": (i32, [i32, i32, vp]),
    "tgk_attn_fwd": (i32, [vp, i32, i32, i32, i32, vp, vp, vp, i32, vp, i32, vp, f32]),
    "tgk_attn_bwd": (i32, [vp, i32, i32, i32, i32, vp, vp, vp, i32, vp, i32, vp, vp, i32, vp, vp, vp, i32,
                           f32, vp, sz]),
    "tgk_attn_bwd_workspace": (sz, [i32, i32, i32]),
    "tgk_attn_bwd_static": (i32, [vp, i32, i32, i32, i32, vp, vp, vp, i32, vp, i32, vp, vp, i32, vp, vp, vp, i32,
                                  f32]),
    "tgk_attn_bwd_static_max_rows": (sz, []),
    "tgk_embed_fwd": (i32, [vp, i32, i32, i32, vp, vp, vp, vp]),
    "tgk_embed_bwd": (i32, [vp, i32, i32, i32, i32, vp, vp, vp, vp, i32, vp, sz]),
    "tgk_embed_bwd_workspace": (sz, [i32, i32]),
    "tgk_embed_bwd_onehot": (i32, [vp, i32, i32, i32, vp, vp, vp, vp, i32]),
    "tgk_layernorm_fwd": (i32, [vp, i32, i32, vp, vp, vp, vp, vp, vp, f32]),
    "tgk_layernorm_bwd": (i32, [vp, i32, i32, vp, vp, vp, vp, vp, vp, vp, f32, i32, i32, vp, sz]),
    "tgk_layernorm_bwd_add": (i32, [vp, i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, f32, i32, vp, sz]),
    "tgk_layernorm_bwd_workspace": (sz, [i32, i32]),
    "tgk_layernorm_bwd_rows": (i32, [vp, i32, i32, vp, vp, vp, vp, vp, vp, f32, vp, sz]),
    "tgk_layernorm_bwd_fold": (i32, [vp, i32, i32, i32, vp, sz, vp, i32]),
    "tgk_cross_entropy": (i32, [vp, i32, i32, vp, vp, vp, vp, f32, i32]),
    "tgk_sumsq_partials": (i32, [vp, vp, sz, vp, i32]),
    "tgk_sumsq_segments": (i32, [vp, vp, vp, i32, vp]),
    "tgk_adamw": (i32, [vp, sz, vp, vp, vp, vp, vp, vp, i32, vp, vp, i32, f32, f32, f32, f32, f32, f32,
                        C.c_uint64]),
    "tgk_sample_batch": (i32, [vp, vp, i64, C.c_uint64, C.c_uint64, i32, i32, vp, vp]),
    "tgk_position_means": (i32, [vp, vp, i32, i32, vp]),
    "tgk_w16_parameter_count": (i32, [i32]),
    "tgk_w16_workspace": (C.c_size_t, [i32, i32, i32]),
    "tgk_w16_forward": (i32, [vp, i32, i32, i32, vp, vp, vp, vp, vp, vp, vp, i32]),
    "tgk_w16_backward": (i32, [vp, i32, i32, i32, vp, vp, vp, vp, vp]),
    "tgk_w16_muon": (i32, [vp, i32, vp, vp, vp, vp, vp, i32, f32, f32, f32, f32, i32]),
}
u64 = C.c_uint64


class Config(C.Structure):
    """config.h:5-13 of the reference; same field order and defaults as tests/bridge.py:7-15."""
    _fields_ = [(x, C.c_int) for x in ("depth", "context", "batch", "device", "blocks", "ns_steps")] + [
        (x, C.c_float) for x in ("learning_rate", "muon_lr", "beta1", "beta2", "momentum", "weight_decay",
                                 "epsilon", "clip")] + [("seed", C.c_uint64), ("inflight", C.c_int)]

    def __init__(self, **kwargs):
        super().__init__(4, 4, 16, 0, 0, 5, .0006, .02, .9, .95, .95, .1, 1e-8, 1., 3407, 1)
        for key, value in kwargs.items():
            setattr(self, key, value)


class WgradJob(C.Structure):
    """TgkWgradJob of include/tgk_kernels.h: one dW[N][K] = dY[M][N]^T X[M][K] of a batch."""
    _fields_ = [("N", C.c_int), ("K", C.c_int), ("dY", C.c_void_p), ("lddy", C.c_int), ("X", C.c_void_p),
                ("ldx", C.c_int), ("dW", C.c_void_p), ("lddw", C.c_int)]


class ModelConfig(C.Structure):
    """TgModelConfig of include/tg_runtime.h: the reference Config plus the model shape."""
    _fields_ = [("base", Config), ("d_model", C.c_int), ("heads", C.c_int), ("vocab", C.c_int), ("ffn", C.c_int),
                ("ln_eps", C.c_float), ("reserved", C.c_int * 3)]

    def __init__(self, d_model=768, heads=None, ffn=None, vocab=256, ln_eps=1e-5, **base):
        super().__init__()
        self.base = Config(**base)
        self.d_model, self.heads = d_model, heads if heads is not None else d_model // 64
        self.vocab, self.ffn, self.ln_eps = vocab, ffn if ffn is not None else 4 * d_model, ln_eps


class OneCycle(C.Structure):
    """optim.h:6-13."""
    _fields_ = [("total_steps", C.c_int)] + [
        (name, C.c_double) for name in ("warmup_fraction", "initial_lr_fraction", "final_lr_fraction",
                                        "low_momentum", "high_momentum")]

    def __init__(self, total_steps, warmup_fraction=.3, initial_lr_fraction=.04, final_lr_fraction=.000004,
                 low_momentum=.85, high_momentum=.95):
        super().__init__(total_steps, warmup_fraction, initial_lr_fraction, final_lr_fraction, low_momentum,
                         high_momentum)


class StepRates(C.Structure):
    _fields_ = [("multiplier", C.c_float), ("momentum", C.c_float)]


# every symbol include/tg_runtime.h declares
ENGINE_ABI = {
    "tg_error": (C.c_char_p, []),
    "tg_create": (vp, [C.POINTER(Config)]),
    "tg_create_ex": (vp, [C.POINTER(ModelConfig)]),
    "tg_destroy": (None, [vp]),
    "tg_parameter_count": (i32, [vp]),
    "tg_blocks": (i32, [vp]),
    "tg_shared_bytes": (i32, [vp]),
    "tg_set_weights": (i32, [vp, vp]),
    "tg_get_weights": (i32, [vp, vp]),
    "tg_get_optimizer_state": (i32, [vp, vp, vp, C.POINTER(u64)]),
    "tg_set_optimizer_state": (i32, [vp, vp, vp, u64]),
    "tg_memory": (i32, [vp, C.POINTER(C.c_double)]),
    "tg_set_data": (i32, [vp, vp, i64]),
    "tg_train": (i32, [vp, i32]),
    "tg_get_training_losses": (i32, [vp, vp, i32]),
    "tg_training_versions": (i32, [vp, vp, i32]),
    "tg_pipeline_stats": (i32, [vp, C.POINTER(C.c_double), C.POINTER(i32)]),
    "tg_onecycle_point": (i32, [C.POINTER(OneCycle), i32, C.POINTER(StepRates)]),
    "tg_set_onecycle": (i32, [vp, C.POINTER(OneCycle)]),
    "tg_batch": (i32, [vp] * 6),
    "tg_predict": (i32, [vp, vp, vp]),
    "tg_optimizer_test": (i32, [vp, vp, i32]),
    "tg_synchronize": (i32, [vp]),
    "tg_profile_step": (i32, [vp, vp, vp, i32]),
}


class Checkpoint(C.Structure):
    """TgCheckpoint of include/tg_checkpoint.h."""
    _fields_ = [("model", ModelConfig), ("parameter_count", i64), ("weights", vp), ("momentum", vp),
                ("variance", vp), ("step", u64), ("scheduler", OneCycle), ("train_seconds", C.c_double),
                ("final_loss_positions", i64), ("final_loss_sums", vp), ("final_loss_batches", u64)]


# every symbol include/tg_checkpoint.h declares
CHECKPOINT_ABI = {
    "tg_checkpoint_write": (i32, [C.c_char_p, C.POINTER(Checkpoint)]),
    "tg_checkpoint_inspect": (i32, [C.c_char_p, C.POINTER(Checkpoint)]),
    "tg_checkpoint_read": (i32, [C.c_char_p, C.POINTER(Checkpoint)]),
    "tg_final_loss_add": (i32, [i32, i32, i32, vp, vp, C.POINTER(u64)]),
}
# every symbol include/tg_events.h declares
EVENTS_ABI = {
    "tg_events_open": (vp, [C.c_char_p, C.c_char_p]),
    "tg_events_path": (C.c_char_p, [vp]),
    "tg_events_scalar": (i32, [vp, C.c_char_p, C.c_double, i64]),
    "tg_events_text": (i32, [vp, C.c_char_p, C.c_char_p, i64]),
    "tg_events_flush": (i32, [vp]),
    "tg_events_close": (i32, [vp]),
    "tg_crc32c": (C.c_uint32, [vp, sz]),
}
CLASSES = ("gemm_fwd", "gemm_dgrad", "gemm_wgrad", "attn_fwd", "attn_bwd", "layernorm_fwd", "layernorm_bwd",
           "head", "other", "optimizer", "gemm_fwd_gelu", "gemm_dgrad_gelu")


def library_path():
    return Path(os.environ.get("TURBOGPT_LIBRARY", str(_HERE / "libturbogpt.so")))


def library():
    """The loaded C-ABI library with argument types declared."""
    global _LIB
    if _LIB is None:
        path = library_path()
        if not path.exists():
            raise RuntimeError(f"{path} is missing: build it with `python -m turbogpt_amd.build` "
                               "(there is no CPU or PyTorch fallback)")
        lib = C.CDLL(str(path))
        for name, (restype, argtypes) in {**KERNEL_ABI, **ENGINE_ABI, **CHECKPOINT_ABI, **EVENTS_ABI}.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.restype, fn.argtypes = restype, argtypes
        _LIB = lib
    return _LIB


def check(status):
    if status < 0:
        raise RuntimeError(library().tg_error().decode())
    return status


class Native:
    """One engine, as in tests/bridge.py:29-81 of the reference: tg_create for a plain Config (the reference's
    width-16 network), tg_create_ex for a ModelConfig."""

    def __init__(self, config):
        import numpy as np
        self.np = np
        self.config = config
        self.lib = library()
        self.base = config if isinstance(config, Config) else config.base
        self.vocab = 256 if isinstance(config, Config) else config.vocab
        create = self.lib.tg_create if isinstance(config, Config) else self.lib.tg_create_ex
        self.handle = create(C.byref(config))
        if not self.handle:
            raise RuntimeError(self.lib.tg_error().decode())
        self.count = self.lib.tg_parameter_count(self.handle)

    def check(self, value):
        if value < 0:
            raise RuntimeError(self.lib.tg_error().decode())

    def close(self):
        if self.handle:
            self.lib.tg_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def set_weights(self, w):
        w = self.np.ascontiguousarray(w, dtype=self.np.float32)
        assert w.size == self.count
        self.check(self.lib.tg_set_weights(self.handle, w.ctypes.data))

    def weights(self):
        w = self.np.empty(self.count, self.np.float32)
        self.check(self.lib.tg_get_weights(self.handle, w.ctypes.data))
        return w

    def optimizer_state(self):
        m, v = self.np.empty(self.count, self.np.float32), self.np.empty(self.count, self.np.float32)
        step = u64()
        self.check(self.lib.tg_get_optimizer_state(self.handle, m.ctypes.data, v.ctypes.data, C.byref(step)))
        return m, v, step.value

    def set_optimizer_state(self, m, v, step):
        m = self.np.ascontiguousarray(m, dtype=self.np.float32)
        v = self.np.ascontiguousarray(v, dtype=self.np.float32)
        self.check(self.lib.tg_set_optimizer_state(self.handle, m.ctypes.data, v.ctypes.data, step))

    def set_data(self, data):
        data = self.np.ascontiguousarray(data, dtype=self.np.uint8)
        self.check(self.lib.tg_set_data(self.handle, data.ctypes.data, data.size))

    def set_onecycle(self, total_steps):
        self.check(self.lib.tg_set_onecycle(self.handle, C.byref(OneCycle(total_steps))))

    def train(self, steps):
        self.check(self.lib.tg_train(self.handle, steps))

    def training_losses(self, count):
        out = self.np.empty((count, self.base.context), self.np.float32)
        self.check(self.lib.tg_get_training_losses(self.handle, out.ctypes.data, count))
        return out

    def optimizer_test(self, grad, steps=1):
        grad = self.np.ascontiguousarray(grad, dtype=self.np.float32)
        assert grad.size == self.count
        self.check(self.lib.tg_optimizer_test(self.handle, grad.ctypes.data, steps))

    def profile_step(self):
        """One training step with per-class HIP-event timing: {class: (milliseconds, launches)}."""
        ms = (C.c_float * len(CLASSES))()
        launches = (C.c_int * len(CLASSES))()
        self.check(self.lib.tg_profile_step(self.handle, ms, launches, len(CLASSES)))
        return {name: (ms[i], launches[i]) for i, name in enumerate(CLASSES)}

    def synchronize(self):
        self.check(self.lib.tg_synchronize(self.handle))

    def batch(self, x, y, backward=True):
        np = self.np
        base = self.base
        x, y = np.ascontiguousarray(x, dtype=np.uint8), np.ascontiguousarray(y, dtype=np.uint8)
        assert x.shape == y.shape == (base.batch, base.context)
        logits = np.empty((*x.shape, self.vocab), np.float32)
        grad = np.empty(self.count, np.float32) if backward else None
        losses = np.empty(base.context, np.float32)
        self.check(self.lib.tg_batch(self.handle, x.ctypes.data, y.ctypes.data, logits.ctypes.data,
                                     grad.ctypes.data if grad is not None else None, losses.ctypes.data))
        return logits, grad, losses

    def predict(self, context):
        np = self.np
        context = np.ascontiguousarray(context, dtype=np.uint8)
        assert context.size == self.base.context
        logits = np.empty(self.vocab, np.float32)
        self.check(self.lib.tg_predict(self.handle, context.ctypes.data, logits.ctypes.data))
        return logits


def write_checkpoint(path, model, weights, momentum, variance, step, scheduler=None, train_seconds=0.0,
                     final_loss_sums=None, final_loss_batches=0):
    """save_training_state of the reference (checkpoint.cpp:554-579) for the target model."""
    import numpy as np
    arrays = [np.ascontiguousarray(a, dtype=np.float32) for a in (weights, momentum, variance)]
    sums = None if final_loss_sums is None else np.ascontiguousarray(final_loss_sums, dtype=np.float64)
    c = Checkpoint()
    c.model = model
    c.parameter_count = arrays[0].size
    c.weights, c.momentum, c.variance = (a.ctypes.data for a in arrays)
    c.step = step
    c.scheduler = scheduler if scheduler is not None else OneCycle(0)
    c.train_seconds = train_seconds
    c.final_loss_positions = 0 if sums is None else sums.size
    c.final_loss_sums = None if sums is None else sums.ctypes.data
    c.final_loss_batches = final_loss_batches
    check(library().tg_checkpoint_write(os.fsencode(path), C.byref(c)))


def read_checkpoint(path, expect=None):
    """load_training_state (checkpoint.cpp:506-551): a dict of the file's contents; `expect`, a
    ModelConfig, makes an architecture mismatch an error."""
    import numpy as np
    lib = library()
    c = Checkpoint()
    check(lib.tg_checkpoint_inspect(os.fsencode(path), C.byref(c)))
    out = {name: np.empty(c.parameter_count, np.float32) for name in ("weights", "momentum", "variance")}
    sums = np.empty(c.final_loss_positions, np.float64)
    c.weights, c.momentum, c.variance = (out[n].ctypes.data for n in ("weights", "momentum", "variance"))
    c.final_loss_sums = sums.ctypes.data if sums.size else None
    if expect is not None:
        c.model = expect
    else:
        c.model.d_model = 0
    check(lib.tg_checkpoint_read(os.fsencode(path), C.byref(c)))
    out.update(step=c.step, train_seconds=c.train_seconds, final_loss_sums=sums,
               final_loss_batches=c.final_loss_batches,
               scheduler={name: getattr(c.scheduler, name) for name, _ in OneCycle._fields_},
               model={"depth": c.model.base.depth, "context": c.model.base.context, "d_model": c.model.d_model,
                      "heads": c.model.heads, "vocab": c.model.vocab, "ffn": c.model.ffn})
    return out
