"""ctypes binding of libpcmi355.so.  There is no fallback: if the library is missing the
import fails with the command that builds it."""
import ctypes
import os

import torch  # noqa: F401  -- first, so that the library binds to the HIP runtime torch has loaded (one runtime per process)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "libpcmi355.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(f"{LIB_PATH} is missing; build it with `python lvd-pg_amd/build.py`")

lib = ctypes.CDLL(LIB_PATH)

c_i32, c_i64, c_f32 = ctypes.c_int32, ctypes.c_int64, ctypes.c_float
vp = ctypes.c_void_p
H = ctypes.c_void_p  # pcm_circuit*

lib.pcm_last_error.restype = ctypes.c_char_p
lib.pcm_version.restype = ctypes.c_int
lib.pcm_size.restype = c_i64
lib.pcm_size.argtypes = [H, c_i32]
lib.pcm_sample_noise_size.restype = c_i64
lib.pcm_sample_noise_size.argtypes = [H]

_SIGS = {
    "pcm_hclt_create": [vp, c_i32, c_i32, c_i32, ctypes.POINTER(H)],
    "pcm_hclt_create_multihead": [vp, c_i32, c_i32, c_i32, c_i32, ctypes.POINTER(H)],
    "pcm_hclt_create_forest": [vp, c_i32, c_i32, c_i32, c_i32, ctypes.POINTER(H)],
    "pcm_set_missing_category": [H, c_i32],
    "pcm_set_soft_reg": [H, c_f32, c_i32, c_i32],
    "pcm_set_flow_scale": [H, c_f32],
    "pcm_hclt_set_heads": [H, vp],
    "pcm_hclt_get_heads": [H, vp],
    "pcm_circuit_create": [c_i32, vp, vp, vp, vp, vp, vp, c_i32, c_i32, c_i32, ctypes.POINTER(H)],
    "pcm_free": [H],
    "pcm_set_stream": [H, vp],
    "pcm_index_table": [H, c_i32, vp, c_i64],
    "pcm_vectorize_parameters": [H, vp, c_i64],
    "pcm_update_parameters": [H, vp, c_i64],
    "pcm_hclt_set_params": [H, vp, vp],
    "pcm_hclt_get_params": [H, vp, vp],
    "pcm_hclt_get_flows": [H, vp, vp],
    "pcm_loglikelihoods": [H, vp, c_i64, c_i64, vp, c_i32, vp],
    "pcm_flows": [H, vp, c_i64, c_i64, vp, c_i32, c_f32, vp, vp],
    "pcm_em_update": [H, c_f32, c_f32],
    "pcm_em_step": [H, vp, c_i64, c_i64, vp, c_i32, c_f32, c_f32, c_f32, vp],
    "pcm_get_node_values": [H, vp, vp, c_i64],
    "pcm_get_aggregates": [H, vp, c_i64, vp, c_i64],
    "pcm_node_flow_sums": [H, vp, c_i64],
    "pcm_kld": [H, H, vp],
    "pcm_kld_backward": [H, H, vp, vp, c_i64],
    "pcm_kld_backward_dev": [H, H, vp, vp, c_i64],
    "pcm_sample": [H, vp, vp, c_i32, vp],
    "pcm_sample_soft": [H, vp, ctypes.c_float, c_i32, vp],
    "pcm_adam_step": [H, vp, vp, vp, vp, c_f32, c_f32, c_f32, c_f32, c_i32],
    "pcm_flow_gradients": [H, c_i32, vp],
    "pcm_adam_flow_step": [H, c_i32, vp, vp, vp, vp, vp, vp, c_f32, c_f32, c_f32, c_f32, c_i32],
    "pcm_kld_rows": [H, vp, vp, c_i64, c_i64, c_i32, c_i32, vp],
    "pcm_kld_backward_rows": [H, vp, vp, c_i64, c_i64, c_i32, c_i32, vp, vp, vp],
    "pcm_gumbel_sample_rows": [H, vp, c_i64, c_i64, c_i32, vp, c_f32, c_i32, vp],
    "pcm_gumbel_sample_backward_rows": [H, vp, c_i64, c_i64, c_i32, vp, c_f32, c_i32, c_i32, vp, vp],
    "pcm_normalized_flows": [H, vp, c_i64, c_i64, vp, c_i32, c_i32, vp, c_i64, c_i64],
    "pcm_normalize_params_rows": [H, vp, c_i64, c_i64, c_i32, c_i32],
    "pcm_stream_probe": [vp, vp, c_i64, c_i32, c_i32, c_i32, vp],
    "pcm_loglikelihoods_soft": [H, vp, c_i64, c_i64, c_i64, vp, c_i32, vp],
    "pcm_flows_soft": [H, vp, c_i64, c_i64, c_i64, vp, c_i32, c_f32, vp, vp],
    "pcm_pairwise_mi": [vp, c_i64, c_i64, c_i64, c_i32, c_i32, c_f32, vp, vp],
    "pcm_pairwise_mi_static": [vp, c_i64, c_i64, c_i64, c_i32, c_i32, c_f32, vp, vp],
    "pcm_chow_liu_tree": [vp, c_i32, vp],
    "pcm_set_timing": [H, c_i32],
    "pcm_get_timing": [H, vp, c_i32],
}
for _name, _args in _SIGS.items():
    _f = getattr(lib, _name)
    _f.argtypes = _args
    _f.restype = ctypes.c_int


class PcmError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"pcmi355 error {status}: {message}")
        self.status = status


def check(status):
    if status != 0:
        raise PcmError(status, lib.pcm_last_error().decode())


def np_ptr(a):
    return None if a is None else a.ctypes.data_as(vp)
