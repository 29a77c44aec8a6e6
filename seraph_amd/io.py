"""ctypes view of include/hip_train_io.h: token files, model directories, checkpoints and
adapter files in the reference's formats.  Pure host code; needs no GPU."""
import ctypes as C

import numpy as np

from ._lib import SeraphError, backend
from .trainer import ModelConfig, lora_param_count, param_count


class TtokFile(C.Structure):
    _fields_ = [("tokens", C.POINTER(C.c_int32)), ("offsets", C.POINTER(C.c_int32)), ("num_samples", C.c_int32),
                ("num_tokens", C.c_int32), ("version", C.c_uint32), ("vocab_size", C.c_uint32)]


class TrainStateFile(C.Structure):
    _fields_ = [("epoch", C.c_int32), ("step", C.c_int32), ("loss", C.c_float), ("optimizer_step", C.c_int32)]


def _lib():
    lib = backend()
    if not getattr(lib, "_seraph_io_bound", False):
        lib.hip_ttok_load.argtypes = [C.c_char_p, C.POINTER(TtokFile)]
        lib.hip_ttok_free.argtypes = [C.POINTER(TtokFile)]
        lib.hip_ttok_write.argtypes = [C.c_char_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_uint32]
        lib.hip_ttok_units.argtypes = [C.POINTER(TtokFile), C.c_int, C.c_int, C.POINTER(C.POINTER(C.c_int32)),
                                       C.POINTER(C.POINTER(C.c_int32))]
        lib.hip_pack_batch.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.POINTER(C.c_int), C.c_int, C.c_int,
                                       C.c_void_p, C.c_void_p, C.POINTER(C.c_int)]
        lib.hip_model_config_load.argtypes = [C.c_char_p, C.POINTER(ModelConfig)]
        lib.hip_weights_load_host.argtypes = [C.c_char_p, C.POINTER(ModelConfig), C.c_void_p, C.POINTER(C.c_int)]
        lib.hip_checkpoint_save_host.argtypes = [C.c_char_p, C.POINTER(ModelConfig), C.c_void_p]
        lib.hip_checkpoint_load_host.argtypes = [C.c_char_p, C.POINTER(ModelConfig), C.c_void_p]
        lib.hip_train_state_save.argtypes = [C.c_char_p, C.POINTER(TrainStateFile)]
        lib.hip_train_state_load.argtypes = [C.c_char_p, C.POINTER(TrainStateFile)]
        lib.hip_lora_init.argtypes = [C.POINTER(ModelConfig), C.c_uint, C.c_void_p]
        lib.hip_lora_save.argtypes = [C.c_char_p, C.POINTER(ModelConfig), C.c_void_p]
        lib.hip_lora_load.argtypes = [C.c_char_p, C.POINTER(ModelConfig), C.c_void_p]
        lib.hip_trainer_load_weights.argtypes = [C.c_void_p, C.POINTER(ModelConfig), C.c_char_p, C.POINTER(C.c_int)]
        lib.hip_trainer_save_checkpoint.argtypes = [C.c_void_p, C.POINTER(ModelConfig), C.c_char_p]
        lib.hip_trainer_load_checkpoint.argtypes = [C.c_void_p, C.POINTER(ModelConfig), C.c_char_p]
        lib.hip_trainer_save_optimizer_state.argtypes = [C.c_void_p, C.c_char_p]
        lib.hip_trainer_load_optimizer_state.argtypes = [C.c_void_p, C.c_char_p]
        lib.free.argtypes = [C.c_void_p]
        lib._seraph_io_bound = True
    return lib


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def ttok_load(path):
    """(tokens int32[n], offsets int32[samples + 1], vocab_size) of a .ttok file."""
    f = TtokFile()
    if _lib().hip_ttok_load(str(path).encode(), C.byref(f)) != 0:
        raise SeraphError(f"cannot load {path} (see stderr)")
    try:
        tokens = np.ctypeslib.as_array(f.tokens, shape=(max(f.num_tokens, 1),))[:f.num_tokens].copy()
        offsets = np.ctypeslib.as_array(f.offsets, shape=(f.num_samples + 1,)).copy()
        return tokens, offsets, int(f.vocab_size)
    finally:
        _lib().hip_ttok_free(C.byref(f))


def ttok_write(path, tokens, offsets, vocab_size):
    tokens = np.ascontiguousarray(tokens, np.int32)
    offsets = np.ascontiguousarray(offsets, np.int32)
    if _lib().hip_ttok_write(str(path).encode(), _ptr(tokens), _ptr(offsets), offsets.size - 1, vocab_size) != 0:
        raise SeraphError(f"cannot write {path}")


def ttok_units(tokens, offsets, max_seq_len, fixed_windows=False):
    """(starts, lengths) of the training units of a token set."""
    tokens = np.ascontiguousarray(tokens, np.int32)
    offsets = np.ascontiguousarray(offsets, np.int32)
    f = TtokFile(tokens.ctypes.data_as(C.POINTER(C.c_int32)), offsets.ctypes.data_as(C.POINTER(C.c_int32)),
                 offsets.size - 1, tokens.size, 1, 0)
    s, l = C.POINTER(C.c_int32)(), C.POINTER(C.c_int32)()
    n = _lib().hip_ttok_units(C.byref(f), max_seq_len, 1 if fixed_windows else 0, C.byref(s), C.byref(l))
    if n < 0:
        raise SeraphError("hip_ttok_units failed")
    try:
        starts = np.ctypeslib.as_array(s, shape=(n + 1,))[:n].copy()
        lengths = np.ctypeslib.as_array(l, shape=(n + 1,))[:n].copy()
    finally:
        _lib().free(s)
        _lib().free(l)
    return starts, lengths


def pack_batches(tokens, starts, lengths, batch_size, max_seq_len):
    """Yields (packed tokens, seq_starts) for one pass over the units, as the trainer front end packs them."""
    tokens = np.ascontiguousarray(tokens, np.int32)
    starts = np.ascontiguousarray(starts, np.int32)
    lengths = np.ascontiguousarray(lengths, np.int32)
    packed = np.empty(batch_size * max_seq_len, np.int32)
    seq = np.empty(batch_size + 1, np.int32)
    idx, total = C.c_int(0), C.c_int(0)
    while True:
        n = _lib().hip_pack_batch(_ptr(tokens), _ptr(starts), _ptr(lengths), starts.size, C.byref(idx), batch_size,
                                  max_seq_len, _ptr(packed), _ptr(seq), C.byref(total))
        if n < 0:
            raise SeraphError("hip_pack_batch failed")
        if n == 0:
            return
        yield packed[:total.value].copy(), seq[:n + 1].copy()


def model_config_load(model_dir):
    cfg = ModelConfig()
    if _lib().hip_model_config_load(str(model_dir).encode(), C.byref(cfg)) != 0:
        raise SeraphError(f"cannot load {model_dir}/config.json (see stderr)")
    return cfg


def weights_load(path, cfg):
    """(parameter arena float32[hip_param_count], number of tensors the files lack)."""
    arena = np.zeros(param_count(cfg), np.float32)
    missing = C.c_int(0)
    if _lib().hip_weights_load_host(str(path).encode(), C.byref(cfg), _ptr(arena), C.byref(missing)) != 0:
        raise SeraphError(f"cannot load weights from {path} (see stderr)")
    return arena, missing.value


def checkpoint_save(path, cfg, arena):
    arena = np.ascontiguousarray(arena, np.float32)
    assert arena.size == param_count(cfg)
    if _lib().hip_checkpoint_save_host(str(path).encode(), C.byref(cfg), _ptr(arena)) != 0:
        raise SeraphError(f"cannot write {path}")


def checkpoint_load(path, cfg):
    arena = np.zeros(param_count(cfg), np.float32)
    if _lib().hip_checkpoint_load_host(str(path).encode(), C.byref(cfg), _ptr(arena)) != 0:
        raise SeraphError(f"cannot load {path} (see stderr)")
    return arena


def train_state_save(checkpoint_path, epoch, step, loss, optimizer_step):
    st = TrainStateFile(epoch, step, loss, optimizer_step)
    if _lib().hip_train_state_save(str(checkpoint_path).encode(), C.byref(st)) != 0:
        raise SeraphError(f"cannot write {checkpoint_path}.state")


def train_state_load(checkpoint_path):
    st = TrainStateFile()
    if _lib().hip_train_state_load(str(checkpoint_path).encode(), C.byref(st)) != 0:
        return None
    return dict(epoch=st.epoch, step=st.step, loss=st.loss, optimizer_step=st.optimizer_step)


def lora_init(cfg, seed):
    arena = np.zeros(lora_param_count(cfg), np.float32)
    if _lib().hip_lora_init(C.byref(cfg), seed, _ptr(arena)) != 0:
        raise SeraphError("hip_lora_init failed")
    return arena


def lora_save(path, cfg, arena):
    arena = np.ascontiguousarray(arena, np.float32)
    assert arena.size == lora_param_count(cfg)
    if _lib().hip_lora_save(str(path).encode(), C.byref(cfg), _ptr(arena)) != 0:
        raise SeraphError(f"cannot write {path}")


def lora_load(path, cfg, arena=None):
    arena = np.zeros(lora_param_count(cfg), np.float32) if arena is None else np.ascontiguousarray(arena, np.float32)
    if _lib().hip_lora_load(str(path).encode(), C.byref(cfg), _ptr(arena)) != 0:
        raise SeraphError(f"cannot load {path} (see stderr)")
    return arena


def trainer_load_weights(trainer, path):
    missing = C.c_int(0)
    if _lib().hip_trainer_load_weights(trainer._h, C.byref(trainer.cfg), str(path).encode(), C.byref(missing)) != 0:
        raise SeraphError(f"cannot load weights from {path} (see stderr)")
    return missing.value


def trainer_save_checkpoint(trainer, path):
    if _lib().hip_trainer_save_checkpoint(trainer._h, C.byref(trainer.cfg), str(path).encode()) != 0:
        raise SeraphError(f"cannot write {path}")


def trainer_load_checkpoint(trainer, path):
    if _lib().hip_trainer_load_checkpoint(trainer._h, C.byref(trainer.cfg), str(path).encode()) != 0:
        raise SeraphError(f"cannot load {path} (see stderr)")


def trainer_save_optimizer_state(trainer, checkpoint_path):
    if _lib().hip_trainer_save_optimizer_state(trainer._h, str(checkpoint_path).encode()) != 0:
        raise SeraphError(f"cannot write {checkpoint_path}.optim")


def trainer_load_optimizer_state(trainer, checkpoint_path):
    """True when the state was loaded, False when <checkpoint>.optim does not exist."""
    rc = _lib().hip_trainer_load_optimizer_state(trainer._h, str(checkpoint_path).encode())
    if rc < 0:
        raise SeraphError(f"cannot load {checkpoint_path}.optim (see stderr)")
    return rc == 0
