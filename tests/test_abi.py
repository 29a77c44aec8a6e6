"""CPU-side checks of the drop-in boundary: both shared libraries load without a GPU and
export every symbol their headers declare; host-side argument validation works without
touching a device."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")

DECL = re.compile(r"^\s*(?:const\s+)?[A-Za-z_][A-Za-z0-9_]*\s*\*?\s*\*?\s*((?:seraph|vulkan|hip)_[a-z0-9_]+)\s*\(", re.M)


def declared(header):
    text = open(os.path.join(INC, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(m for m in DECL.findall(text)))


@pytest.fixture(scope="module")
def libs():
    from seraph_amd import _lib
    if not os.path.exists(_lib.KERNEL_LIB) or not os.path.exists(_lib.BACKEND_LIB):
        from seraph_amd import build
        build.build_all()
    return _lib.kernels(), _lib.backend()


def test_kernel_library_exports_its_header(libs):
    k, _ = libs
    names = declared("seraph_hip.h")
    assert len(names) >= 40
    missing = [n for n in names if not hasattr(k, n)]
    assert not missing, missing


def test_backend_exports_the_reference_api_and_additions(libs):
    _, b = libs
    names = declared("hip_backend.h") + declared("hip_train.h") + declared("hip_train_io.h")
    assert "hip_ttok_load" in names and "hip_eval_forward_batch" in names and "hip_trainer_nan_flags" in names
    missing = [n for n in names if not hasattr(b, n)]
    assert not missing, missing
    # the 40 symbols an unmodified train.o leaves undefined (nm -u on the reference object)
    needed = """vulkan_init_ex vulkan_free vulkan_cmd_begin vulkan_cmd_end_submit vulkan_buffer_create vulkan_buffer_free
    vulkan_buffer_upload vulkan_buffer_upload_u32 vulkan_buffer_download vulkan_buffer_download_bytes vulkan_fill_buffer
    vulkan_fill_buffer_range vulkan_copy_buffer vulkan_copy_buffer_cache vulkan_barrier_transfer_to_compute
    vulkan_nan_check vulkan_matmul vulkan_matmul_transpose vulkan_adamw_update vulkan_add vulkan_mul vulkan_scale
    vulkan_silu vulkan_rmsnorm vulkan_rope vulkan_batch_attention vulkan_embed_lookup vulkan_cross_entropy_grad
    vulkan_reduce_sum vulkan_rmsnorm_backward_batch vulkan_rope_backward vulkan_batch_attention_backward
    vulkan_embedding_backward vulkan_silu_backward vulkan_elementwise_mul_backward vulkan_qk_norm vulkan_patch_extract
    vulkan_add_bias vulkan_bce_loss_grad vulkan_sum_cols""".split()
    assert len(needed) == 40
    assert not [n for n in needed if not hasattr(b, n)]


def test_argument_validation_needs_no_device(libs):
    k, _ = libs
    k.seraph_hip_last_error.restype = C.c_char_p
    assert k.seraph_gemm(None, None, None, C.c_int64(4), C.c_int64(4), C.c_int64(4), 0, 0, 0, None) == -1
    assert b"NULL" in k.seraph_hip_last_error()
    assert k.seraph_adamw(None, None, None, None, C.c_size_t(0), C.c_float(0), C.c_float(0), C.c_float(0),
                          C.c_float(0), C.c_float(0), 1, C.c_float(0), None) == 0           # empty tensor: no-op
    k.seraph_attention_backward_ws_bytes.restype = C.c_size_t
    assert k.seraph_attention_backward_ws_bytes(C.c_int64(1024), 16, 8, 128) >= 1024 * 16 * 128 * 4
    # the norm backward in two halves: an empty pass reports no partial rows, a missing scratch is refused before
    # any launch, an empty job list is a no-op and a list without its array is an error
    n = C.c_int(7)
    assert k.seraph_rmsnorm_backward_rows(None, None, None, None, None, C.c_int64(0), C.c_int64(512), C.c_float(1e-5),
                                          None, C.c_size_t(0), C.byref(n), None) == 0 and n.value == 0
    p = C.c_void_p(256)                                  # never dereferenced: the scratch check comes first
    assert k.seraph_rmsnorm_backward_rows(p, p, p, None, p, C.c_int64(64), C.c_int64(512), C.c_float(1e-5),
                                          None, C.c_size_t(0), C.byref(n), None) == -3
    assert b"scratch" in k.seraph_hip_last_error()
    assert k.seraph_rmsnorm_colsum_multi(None, 0, C.c_int64(512), None) == 0
    assert k.seraph_rmsnorm_colsum_multi(None, 3, C.c_int64(512), None) == -1


def test_param_count_matches_reference_shapes(libs):
    from seraph_amd import trainer
    # Seraph-native 33M model (tied embeddings): 8192*512 + 512 + 8*(2*512 + 4*512*512 + 3*512*1408)
    c1 = trainer.model_config(512, 8, 8, 8, 64, 1408, 8192)
    assert trainer.param_count(c1) == 8192 * 512 + 512 + 8 * (2 * 512 + 4 * 512 * 512 + 3 * 512 * 1408)
    # Qwen3-1.7B shape: 1.72 G parameters
    c5 = trainer.model_config(2048, 28, 16, 8, 128, 6144, 151936)
    n = trainer.param_count(c5)
    assert n == 151936 * 2048 + 2048 + 28 * (2 * 2048 + 2 * 2048 * 2048 + 2 * 1024 * 2048 + 3 * 2048 * 6144)
    lora = trainer.model_config(2048, 28, 16, 8, 128, 6144, 151936, lora_rank=16, lora_alpha=32.0, lora_mask=15)
    assert trainer.lora_param_count(lora) == 28 * 16 * ((2048 + 2048) + 2 * (2048 + 1024) + (2048 + 2048))


def test_bench_refuses_more_than_one_gpu():
    """The build is for one GPU: --gpus N > 1 ends with a message, not with a number."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert p.returncode != 0 and "one GPU" in (p.stdout + p.stderr)
    assert '"metric"' not in p.stdout
