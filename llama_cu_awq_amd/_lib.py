"""ctypes binding of libawq_hip.so.  The library is the product: if it cannot be loaded this module raises."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
lib_path = os.path.join(_HERE, "libawq_hip.so")


class AwqError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"libawq_hip status {code}: {text}")
        self.code = code


class QWeightC(C.Structure):
    _fields_ = [("weight", C.c_void_p), ("zeros", C.c_void_p), ("scales", C.c_void_p)]


class ConfigC(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads", "vocab_size", "seq_len")] + [
        ("rope_theta", C.c_float)
    ]


class RunStateC(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("x", "xb", "hb", "q", "att", "logits", "key_cache", "value_cache", "pos", "shared_pos", "shared_tokens")]


class LayerWeightsC(C.Structure):
    _fields_ = [("rms_att_weight", C.c_void_p), ("rms_ffn_weight", C.c_void_p)] + [
        (n, QWeightC) for n in ("wq_q", "wq_k", "wq_v", "wq_o", "wq_gate", "wq_up", "wq_down")
    ]


AWQ_OK, AWQ_ERR_ARG, AWQ_ERR_SHAPE, AWQ_ERR_HIP, AWQ_ERR_IO = 0, -1, -2, -3, -4

_vp, _i, _sz, _f = C.c_void_p, C.c_int, C.c_size_t, C.c_float
_pvp = C.POINTER(C.c_void_p)
_pq = C.POINTER(QWeightC)

# name -> argtypes; every function returns int except the two noted below
PROTOTYPES = {
    "awq_device_count": [C.POINTER(C.c_int)],
    "awq_device_info": [_i, C.c_char_p, _sz, C.POINTER(C.c_size_t), C.POINTER(C.c_int)],
    "awq_ctx_create": [_i, _pvp],
    "awq_ctx_create_on_stream": [_i, _vp, _pvp],
    "awq_ctx_destroy": [_vp],
    "awq_stream_sync": [_vp],
    "awq_malloc": [_vp, _pvp, _sz],
    "awq_free": [_vp, _vp],
    "awq_malloc_host": [_vp, _pvp, _sz],
    "awq_free_host": [_vp, _vp],
    "awq_memcpy_h2d_async": [_vp, _vp, _vp, _sz],
    "awq_memcpy_h2d": [_vp, _vp, _vp, _sz],
    "awq_memcpy_d2h": [_vp, _vp, _vp, _sz],
    "awq_memcpy_d2d_async": [_vp, _vp, _vp, _sz],
    "awq_memset_async": [_vp, _vp, _i, _sz],
    "awq_event_create": [_vp, _pvp],
    "awq_event_destroy": [_vp, _vp],
    "awq_event_record": [_vp, _vp],
    "awq_event_elapsed_ms": [_vp, _vp, _vp, C.POINTER(C.c_float)],
    "awq_embed": [_vp, _vp, _vp, _i, _vp, _vp],
    "awq_rmsnorm": [_vp, _vp, _vp, _vp, _i],
    "awq_matvec_int4": [_vp, _vp, _vp, _pq, _i, _i, _i, _i, _i, _vp],
    "awq_qkv_matvec": [_vp, _vp, _vp, _vp, _vp, _pq, _pq, _pq, _i, _i, _i, _vp],
    "awq_ffn_matvec_silu": [_vp, _vp, _vp, _pq, _pq, _i, _i],
    "awq_rmsnorm_ffn_matvec_silu": [_vp, _vp, _vp, _vp, _pq, _pq, _i, _i],
    "awq_rope": [_vp, _vp, _vp, _i, _i, _i, _vp, _i, _f],
    "awq_attention": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "awq_attention_partial": [_vp, _vp, C.POINTER(C.c_int), _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "awq_matvec_int4_parts": [_vp, _vp, _vp, _i, _pq, _i, _i, _i],
    "awq_matvec_f16": [_vp, _vp, _vp, _vp, _i, _i],
    "awq_argmax_advance": [_vp, _vp, _i, _vp, _vp, _vp, _i],
    "awq_dequant": [_vp, _vp, _pq, _i, _i],
    "awq_transformer_load_file": [_vp, C.c_char_p, _pvp],
    "awq_transformer_load_image": [_vp, _vp, _sz, _pvp],
    "awq_transformer_free": [_vp],
    "awq_transformer_config": [_vp, C.POINTER(ConfigC)],
    "awq_transformer_state": [_vp, C.POINTER(RunStateC)],
    "awq_transformer_layer": [_vp, _i, C.POINTER(LayerWeightsC)],
    "awq_transformer_globals": [_vp, _pvp, _pvp, _pvp],
    "awq_transformer_reset": [_vp, C.POINTER(C.c_int), _i],
    "awq_transformer_set_pos": [_vp, _i, _i],
    "awq_transformer_forward": [_vp, _i, _i, _i],
    "awq_transformer_capture": [_vp, _i, _i],
    "awq_transformer_time_launches": [_vp, _i, C.POINTER(C.c_float), C.POINTER(C.c_int)],
    "awq_gemm_int4": [_vp, _vp, _i, _vp, _i, _i, _pq, _i, _i, _i],
    "awq_gemm_int4_static": [_vp, _vp, _i, _vp, _i, _i, _pq, _i, _i, _i],
    "awq_transformer_prefill": [_vp, _i, _i],
    "awq_transformer_forward_logits": [_vp, _i, _i],
    "awq_transformer_accept": [_vp, _i, _i],
    "awq_transformer_trace": [_vp, _i, C.POINTER(C.c_longlong), _i, C.POINTER(C.c_int)],
    "awq_softmax_logits": [_vp, _vp, _i, _f],
    "awq_sample_top_p": [_vp, _vp, _i, _f, _i, _vp, _vp, _vp],
    "awq_sampler_create": [_vp, _i, _f, _f, C.c_ulonglong, _pvp],
    "awq_sampler_destroy": [_vp],
    "awq_sampler_sample": [_vp, _vp, _vp, _vp, _vp, _i],
    "awq_transformer_sample": [_vp, _vp, _i],
}
NON_STATUS = {"awq_last_error": ([], C.c_char_p), "awq_ctx_stream": ([_vp], _vp)}


def _load():
    if not os.path.exists(lib_path):
        raise ImportError(
            f"{lib_path} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(or __graft_entry__.build()); there is no fallback path"
        )
    h = C.CDLL(lib_path)
    for name, args in PROTOTYPES.items():
        fn = getattr(h, name)
        fn.argtypes = args
        fn.restype = C.c_int
    for name, (args, res) in NON_STATUS.items():
        fn = getattr(h, name)
        fn.argtypes = args
        fn.restype = res
    return h


lib = _load()


def check(status):
    if status != AWQ_OK:
        raise AwqError(status, lib.awq_last_error().decode(errors="replace"))
