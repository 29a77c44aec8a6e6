"""Python handle on the packed-batch training steps of libseraph_hip_backend.so
(include/hip_train.h).  Mirrors cuda_train_step_gpu_full_batch / ..._lora_batch of the
reference (include/train_cuda.h:41-49): a packed token stream plus seq_starts in, mean
loss out; parameters, gradients and Adam moments stay on the device."""
import ctypes as C

import numpy as np

from ._lib import SeraphError, backend


class ModelConfig(C.Structure):
    _fields_ = [("hidden", C.c_int32), ("layers", C.c_int32), ("heads", C.c_int32), ("kv_heads", C.c_int32),
                ("head_dim", C.c_int32), ("ffn", C.c_int32), ("vocab", C.c_int32), ("rms_eps", C.c_float),
                ("rope_theta", C.c_float), ("lora_rank", C.c_int32), ("lora_alpha", C.c_float),
                ("lora_mask", C.c_int32), ("use_qk_norm", C.c_int32)]


class OptimConfig(C.Structure):
    _fields_ = [("learning_rate", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float),
                ("weight_decay", C.c_float), ("eps", C.c_float), ("clip", C.c_float),
                ("warmup_steps", C.c_int32), ("gradient_accumulation_steps", C.c_int32)]


class OpStat(C.Structure):
    _fields_ = [("name", C.c_char_p), ("launches", C.c_int64), ("ms", C.c_double), ("flops", C.c_double),
                ("bytes", C.c_double)]


class ParamLayout(C.Structure):
    _fields_ = [(n, C.c_int64) for n in ("embed", "final_norm", "layer0", "layer_stride", "in_norm", "q", "k", "v", "o",
                                         "post_norm", "gate", "up", "down", "count")]


class LoraLayout(C.Structure):
    _fields_ = [("A", C.c_int64 * 7), ("B", C.c_int64 * 7), ("in_dim", C.c_int64 * 7), ("out_dim", C.c_int64 * 7),
                ("layer_stride", C.c_int64), ("count", C.c_int64)]


PARAMS, GRADS, ADAM_M, ADAM_V, LORA_PARAMS, LORA_GRADS, LORA_M, LORA_V = range(8)


def model_config(hidden, layers, heads, kv_heads, head_dim, ffn, vocab, rms_eps=1e-5, rope_theta=10000.0,
                 lora_rank=0, lora_alpha=0.0, lora_mask=0, use_qk_norm=0):
    return ModelConfig(hidden, layers, heads, kv_heads, head_dim, ffn, vocab, rms_eps, rope_theta, lora_rank,
                       lora_alpha, lora_mask, use_qk_norm)


def optim_config(learning_rate, beta1=0.9, beta2=0.999, weight_decay=0.01, eps=1e-8, clip=0.0, warmup_steps=100,
                 gradient_accumulation_steps=1):
    return OptimConfig(learning_rate, beta1, beta2, weight_decay, eps, clip, warmup_steps, gradient_accumulation_steps)


def _lib():
    lib = backend()
    if not getattr(lib, "_seraph_train_bound", False):
        lib.hip_param_count.restype = C.c_int64
        lib.hip_lora_param_count.restype = C.c_int64
        lib.hip_trainer_create.restype = C.c_void_p
        lib.hip_trainer_create.argtypes = [C.POINTER(ModelConfig), C.POINTER(OptimConfig), C.c_int, C.c_int, C.c_int,
                                           C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        lib.hip_trainer_free.argtypes = [C.c_void_p]
        lib.hip_trainer_upload.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int64]
        lib.hip_trainer_download.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int64]
        lib.hip_trainer_device_ptr.restype = C.c_void_p
        lib.hip_trainer_device_ptr.argtypes = [C.c_void_p, C.c_int]
        for f in (lib.hip_train_step_full_batch, lib.hip_train_step_lora_batch):
            f.restype = C.c_float
            f.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int]
        lib.hip_trainer_optimizer_step.argtypes = [C.c_void_p]
        lib.hip_trainer_last_lr.restype = C.c_float
        lib.hip_trainer_last_lr.argtypes = [C.c_void_p]
        lib.hip_trainer_last_timing.argtypes = [C.c_void_p, C.POINTER(C.c_float * 3)]
        lib.hip_trainer_device_bytes.restype = C.c_size_t
        lib.hip_trainer_device_bytes.argtypes = [C.c_void_p]
        lib.hip_trainer_enable_op_timing.argtypes = [C.c_void_p, C.c_int]
        lib.hip_trainer_enable_wgrad_overlap.argtypes = [C.c_void_p, C.c_int]
        lib.hip_trainer_enable_wgrad_overlap.restype = None
        lib.hip_trainer_reset_op_stats.argtypes = [C.c_void_p]
        lib.hip_trainer_op_stats.argtypes = [C.c_void_p, C.POINTER(OpStat), C.c_int]
        lib.hip_trainer_upload_at.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_void_p, C.c_int64]
        lib.hip_trainer_download_at.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_void_p, C.c_int64]
        lib.hip_trainer_arena_count.restype = C.c_int64
        lib.hip_trainer_arena_count.argtypes = [C.c_void_p, C.c_int]
        lib.hip_eval_forward_batch.restype = C.c_float
        lib.hip_eval_forward_batch.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int]
        lib.hip_evaluate.restype = C.c_float
        lib.hip_evaluate.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                     C.POINTER(C.c_float)]
        lib.hip_trainer_set_schedule.argtypes = [C.c_void_p, C.c_float, C.c_int, C.c_int]
        lib.hip_trainer_accumulation_counter.argtypes = [C.c_void_p]
        lib.hip_trainer_enable_nan_check.argtypes = [C.c_void_p, C.c_int]
        lib.hip_trainer_nan_detected.argtypes = [C.c_void_p]
        lib.hip_trainer_set_nan_dump_prefix.argtypes = [C.c_void_p, C.c_char_p]
        lib.hip_trainer_nan_flags.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        lib.hip_param_layout.argtypes = [C.POINTER(ModelConfig), C.POINTER(ParamLayout)]
        lib.hip_lora_layout.argtypes = [C.POINTER(ModelConfig), C.POINTER(LoraLayout)]
        lib._seraph_train_bound = True
    return lib


def param_count(cfg):
    return int(_lib().hip_param_count(C.byref(cfg)))


def lora_param_count(cfg):
    return int(_lib().hip_lora_param_count(C.byref(cfg)))


def param_layout(cfg):
    out = ParamLayout()
    _lib().hip_param_layout(C.byref(cfg), C.byref(out))
    return out


def lora_layout(cfg):
    out = LoraLayout()
    _lib().hip_lora_layout(C.byref(cfg), C.byref(out))
    return out


class Trainer:
    def __init__(self, cfg, opt, max_tokens, max_batch, device=0, ext=(None, None, None, None)):
        self.cfg, self.opt = cfg, opt
        self.lora = cfg.lora_rank > 0
        self._ext = ext                      # keep caller-owned arenas alive
        ptrs = [C.c_void_p(t.data_ptr()) if t is not None else None for t in ext]
        self._h = _lib().hip_trainer_create(C.byref(cfg), C.byref(opt), max_tokens, max_batch, device, *ptrs)
        if not self._h:
            raise SeraphError("hip_trainer_create failed (see stderr)")
        self.nparams = param_count(cfg)
        self.nlora = lora_param_count(cfg)

    def close(self):
        if self._h:
            _lib().hip_trainer_free(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def _count(self, which):
        return self.nparams if which < 4 else self.nlora

    def upload(self, which, host):
        host = np.ascontiguousarray(host, np.float32)
        if _lib().hip_trainer_upload(self._h, which, host.ctypes.data_as(C.c_void_p), host.size) != 0:
            raise SeraphError(f"upload of arena {which} failed (size {host.size}, expected {self._count(which)})")

    def download(self, which):
        out = np.empty(self._count(which), np.float32)
        if _lib().hip_trainer_download(self._h, which, out.ctypes.data_as(C.c_void_p), out.size) != 0:
            raise SeraphError(f"download of arena {which} failed")
        return out

    def step(self, tokens, seq_starts=None, run_optimizer=True):
        tokens = np.ascontiguousarray(tokens, np.int32)
        batch = 1
        sp = None
        if seq_starts is not None:
            seq_starts = np.ascontiguousarray(seq_starts, np.int32)
            batch = seq_starts.size - 1
            sp = seq_starts.ctypes.data_as(C.c_void_p)
        fn = _lib().hip_train_step_lora_batch if self.lora else _lib().hip_train_step_full_batch
        loss = fn(self._h, tokens.ctypes.data_as(C.c_void_p), tokens.size, sp, batch, 1 if run_optimizer else 0)
        if loss < 0:
            raise SeraphError("training step failed (see stderr)")
        return float(loss)

    def eval_forward(self, tokens, seq_starts=None):
        """Forward and loss only (cuda_eval_forward of the reference); changes no state."""
        tokens = np.ascontiguousarray(tokens, np.int32)
        batch, sp = 1, None
        if seq_starts is not None:
            seq_starts = np.ascontiguousarray(seq_starts, np.int32)
            batch = seq_starts.size - 1
            sp = seq_starts.ctypes.data_as(C.c_void_p)
        return float(_lib().hip_eval_forward_batch(self._h, tokens.ctypes.data_as(C.c_void_p), tokens.size, sp, batch))

    def evaluate(self, val_tokens, offsets, max_seq_len, max_eval_samples=0):
        """(mean loss, perplexity) over a validation set, sample by sample (cuda_evaluate of the reference)."""
        val_tokens = np.ascontiguousarray(val_tokens, np.int32)
        offsets = np.ascontiguousarray(offsets, np.int32)
        ppl = C.c_float(0.0)
        loss = _lib().hip_evaluate(self._h, val_tokens.ctypes.data_as(C.c_void_p), val_tokens.size,
                                   offsets.ctypes.data_as(C.c_void_p), offsets.size - 1, max_seq_len, max_eval_samples,
                                   C.byref(ppl))
        return float(loss), float(ppl.value)

    def set_schedule(self, learning_rate, optimizer_step=-1, accumulation_counter=-1):
        _lib().hip_trainer_set_schedule(self._h, learning_rate, optimizer_step, accumulation_counter)

    @property
    def accumulation_counter(self):
        return int(_lib().hip_trainer_accumulation_counter(self._h))

    def enable_nan_check(self, on=True):
        if _lib().hip_trainer_enable_nan_check(self._h, 1 if on else 0) != 0:
            raise SeraphError("could not allocate the NaN flags")

    def set_nan_dump_prefix(self, prefix):
        """Where a step that detects a NaN/Inf writes its buffers ("<prefix>_<step>_<name>"); None: nowhere."""
        _lib().hip_trainer_set_nan_dump_prefix(self._h, prefix.encode() if prefix else None)

    @property
    def nan_detected(self):
        return bool(_lib().hip_trainer_nan_detected(self._h))

    def nan_flags(self):
        n = _lib().hip_trainer_nan_flags(self._h, None, 0)
        out = np.zeros(n, np.uint32)
        _lib().hip_trainer_nan_flags(self._h, out.ctypes.data_as(C.c_void_p), n)
        return out

    @property
    def optimizer_step(self):
        return int(_lib().hip_trainer_optimizer_step(self._h))

    @property
    def last_lr(self):
        return float(_lib().hip_trainer_last_lr(self._h))

    def last_timing(self):
        ms = (C.c_float * 3)()
        _lib().hip_trainer_last_timing(self._h, C.byref(ms))
        return {"forward_loss_ms": ms[0], "backward_ms": ms[1], "optimizer_ms": ms[2]}

    def enable_op_timing(self, on=True):
        _lib().hip_trainer_enable_op_timing(self._h, 1 if on else 0)

    def enable_wgrad_overlap(self, on=True):
        """Weight gradients on a second stream beside the input-gradient chain (full-weight mode; on by default)."""
        _lib().hip_trainer_enable_wgrad_overlap(self._h, 1 if on else 0)

    def reset_op_stats(self):
        _lib().hip_trainer_reset_op_stats(self._h)

    def op_stats(self):
        """Per kernel class: launches, summed device ms, summed algorithmic flops / bytes."""
        buf = (OpStat * 64)()
        n = _lib().hip_trainer_op_stats(self._h, buf, 64)
        return [dict(name=buf[i].name.decode(), launches=int(buf[i].launches), ms=buf[i].ms, flops=buf[i].flops,
                     bytes=buf[i].bytes) for i in range(n)]

    @property
    def device_bytes(self):
        return int(_lib().hip_trainer_device_bytes(self._h))
