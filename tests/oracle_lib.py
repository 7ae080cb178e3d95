"""ctypes bindings for the CPU oracle (oracle/libcpu_ref.so) and, where it was built, the
compiled reference trainer (oracle/_ref/libtrain_gpt2_ref.so).

Test infrastructure only: nothing in the shipped package imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
CREF_SO = os.path.join(ORACLE_DIR, "libcpu_ref.so")
REF_SO = os.path.join(ORACLE_DIR, "_ref", "libtrain_gpt2_ref.so")

f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")
u32p = np.ctypeslib.ndpointer(dtype=np.uint32, flags="C_CONTIGUOUS")


class Config(C.Structure):
    _fields_ = [(n, C.c_int) for n in
                ("max_seq_len", "vocab_size", "padded_vocab_size", "num_layers", "num_heads", "channels")]


def _opt(arr):
    """ndarray -> void* (None -> NULL)"""
    return None if arr is None else arr.ctypes.data_as(C.c_void_p)


def build_cref():
    subprocess.run(["make", "-s", "-C", ORACLE_DIR, "all"], check=True)


_cref = None
_ref = None


def cref():
    """The repo's CPU restatement. Built on demand (gcc only)."""
    global _cref
    if _cref is not None:
        return _cref
    if not os.path.exists(CREF_SO):
        build_cref()
    L = C.CDLL(CREF_SO)
    L.cref_f32_to_bf16_array.argtypes = [u16p, f32p, C.c_size_t]
    L.cref_bf16_to_f32_array.argtypes = [f32p, u16p, C.c_size_t]
    L.cref_f32_to_bf16.argtypes = [C.c_float]
    L.cref_f32_to_bf16.restype = C.c_uint16
    L.cref_mt_kat.argtypes = [C.c_uint32, u32p, f32p, u32p, f32p, u32p]
    L.cref_param_sizes.argtypes = [np.ctypeslib.ndpointer(dtype=np.uint64), C.POINTER(Config)]
    L.cref_param_sizes.restype = C.c_size_t
    L.cref_init_params.argtypes = [f32p, C.POINTER(Config), C.c_uint32]
    L.cref_write_checkpoint_fp32.argtypes = [C.c_char_p, f32p, C.POINTER(Config)]
    L.cref_write_checkpoint_fp32.restype = C.c_int
    L.cref_encoder_forward.argtypes = [f32p, i32p, f32p, f32p, C.c_int, C.c_int, C.c_int]
    L.cref_encoder_backward.argtypes = [f32p, f32p, f32p, i32p, C.c_int, C.c_int, C.c_int]
    L.cref_layernorm_forward.argtypes = [f32p, C.c_void_p, C.c_void_p, f32p, f32p, f32p, C.c_int, C.c_int]
    L.cref_layernorm_backward.argtypes = [f32p, f32p, f32p, f32p, f32p, f32p, f32p, f32p, C.c_int, C.c_int]
    L.cref_matmul_forward.argtypes = [f32p, f32p, f32p, C.c_void_p, C.c_int, C.c_int, C.c_int]
    L.cref_matmul_backward.argtypes = [C.c_void_p, f32p, C.c_void_p, f32p, f32p, f32p, C.c_int, C.c_int, C.c_int]
    L.cref_attention_forward.argtypes = [f32p, C.c_void_p, C.c_void_p, f32p, C.c_int, C.c_int, C.c_int, C.c_int]
    L.cref_attention_backward.argtypes = [f32p, f32p, f32p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int]
    L.cref_gelu_forward.argtypes = [f32p, f32p, C.c_size_t]
    L.cref_gelu_backward.argtypes = [f32p, f32p, f32p, C.c_size_t]
    L.cref_residual_forward.argtypes = [f32p, f32p, f32p, C.c_size_t]
    L.cref_softmax_crossentropy_forward.argtypes = [f32p, C.c_void_p, f32p, C.c_void_p, C.c_int, C.c_int, C.c_int]
    L.cref_crossentropy_softmax_backward.argtypes = [f32p, f32p, i32p, C.c_float, C.c_int, C.c_int, C.c_int]
    L.cref_adamw.argtypes = [f32p, f32p, f32p, f32p, C.c_size_t] + [C.c_float] * 5 + [C.c_int]
    L.cref_sum_squares.argtypes = [f32p, C.c_size_t]
    L.cref_sum_squares.restype = C.c_double
    L.cref_squirrel_noise5.argtypes = [C.c_uint32, C.c_uint32]
    L.cref_squirrel_noise5.restype = C.c_uint32
    L.cref_noise_2d.argtypes = [C.c_int, C.c_int, C.c_uint32]
    L.cref_noise_2d.restype = C.c_uint32
    L.cref_stochastic_round_bf16.argtypes = [C.c_float, C.c_uint32]
    L.cref_stochastic_round_bf16.restype = C.c_uint16
    L.cref_adamw_noise.argtypes = [C.c_size_t, C.c_int, C.c_uint32]
    L.cref_adamw_noise.restype = C.c_uint32
    L.cref_adamw_mixed.argtypes = [u16p, C.c_void_p, u16p, f32p, f32p, C.c_size_t, C.c_float, C.c_float, C.c_float,
                                   C.c_int, C.c_float, C.c_float, C.c_float, C.c_uint32, C.c_int]
    L.cref_adamw_f32.argtypes = [f32p, C.c_void_p, f32p, f32p, f32p, C.c_size_t, C.c_float, C.c_float, C.c_float,
                                 C.c_int, C.c_float, C.c_float, C.c_float]
    L.cref_random_u32.argtypes = [C.POINTER(C.c_uint64)]
    L.cref_random_u32.restype = C.c_uint32
    L.cref_gpt2_train.argtypes = [C.POINTER(Config), f32p, i32p, i32p, C.c_int, C.c_int, C.c_int,
                                  C.c_float, C.c_float, C.c_float, C.c_float, C.c_float, C.c_float, C.c_int,
                                  f32p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
    L.cref_gpt2_train.restype = C.c_int
    L.cref_random_f32.argtypes = [C.POINTER(C.c_uint64)]
    L.cref_random_f32.restype = C.c_float
    L.cref_sample_softmax.argtypes = [f32p, C.c_int, C.c_float]
    L.cref_sample_softmax.restype = C.c_int
    L.cref_gpt2_logits.argtypes = [C.POINTER(Config), f32p, i32p, C.c_int, C.c_int, f32p]
    L.cref_gpt2_logits.restype = C.c_int
    L.cref_gpt2_generate.argtypes = [C.POINTER(Config), f32p, i32p, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_uint64)]
    L.cref_gpt2_generate.restype = C.c_int
    L.cref_num_threads.restype = C.c_int
    _cref = L
    return L


def have_ref():
    return os.path.exists(REF_SO)


def ref():
    """The reference's own train_gpt2.c compiled as a shared object (prebuilt; see oracle/Makefile)."""
    global _ref
    if _ref is not None:
        return _ref
    L = C.CDLL(REF_SO)
    L.encoder_forward.argtypes = [f32p, i32p, f32p, f32p, C.c_int, C.c_int, C.c_int]
    L.encoder_backward.argtypes = [f32p, f32p, f32p, i32p, C.c_int, C.c_int, C.c_int]
    L.layernorm_forward.argtypes = [f32p, f32p, f32p, f32p, f32p, f32p, C.c_int, C.c_int, C.c_int]
    L.layernorm_backward.argtypes = [f32p] * 8 + [C.c_int] * 3
    L.matmul_forward.argtypes = [f32p, f32p, f32p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int]
    L.matmul_forward_naive.argtypes = L.matmul_forward.argtypes
    L.matmul_backward.argtypes = [f32p, f32p, C.c_void_p, f32p, f32p, f32p, C.c_int, C.c_int, C.c_int, C.c_int]
    L.attention_forward.argtypes = [f32p, f32p, f32p, f32p, C.c_int, C.c_int, C.c_int, C.c_int]
    L.attention_backward.argtypes = [f32p] * 6 + [C.c_int] * 4
    L.gelu_forward.argtypes = [f32p, f32p, C.c_int]
    L.gelu_backward.argtypes = [f32p, f32p, f32p, C.c_int]
    L.residual_forward.argtypes = [f32p, f32p, f32p, C.c_int]
    L.softmax_forward.argtypes = [f32p, f32p, C.c_int, C.c_int, C.c_int, C.c_int]
    L.crossentropy_forward.argtypes = [f32p, f32p, i32p, C.c_int, C.c_int, C.c_int]
    L.crossentropy_softmax_backward.argtypes = [f32p, f32p, f32p, i32p, C.c_int, C.c_int, C.c_int, C.c_int]
    L.ref_mt_kat.argtypes = [C.c_uint32, u32p, f32p, u32p, f32p, u32p]
    L.ref_gpt2_train.argtypes = [C.c_char_p, i32p, i32p, C.c_int, C.c_int, C.c_int,
                                 C.c_float, C.c_float, C.c_float, C.c_float, C.c_float,
                                 f32p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
    L.ref_gpt2_train.restype = C.c_int
    L.random_f32.argtypes = [C.POINTER(C.c_uint64)]
    L.random_f32.restype = C.c_float
    L.sample_softmax.argtypes = [f32p, C.c_int, C.c_float]
    L.sample_softmax.restype = C.c_int
    L.ref_gpt2_generate.argtypes = [C.c_char_p, i32p, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_uint64)]
    L.ref_gpt2_generate.restype = C.c_int
    szp = np.ctypeslib.ndpointer(dtype=np.uint64, flags="C_CONTIGUOUS")
    L.ref_dataloader_run.argtypes = [C.c_char_p, C.c_size_t, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                     i32p, i32p, szp, szp, C.POINTER(C.c_size_t), C.c_void_p]
    L.ref_dataloader_run.restype = C.c_size_t
    L.ref_evalloader_run.argtypes = [C.c_char_p, C.c_size_t, C.c_size_t, C.c_int, C.c_int, C.c_int, i32p, i32p,
                                     np.ctypeslib.ndpointer(dtype=np.int8, flags="C_CONTIGUOUS"), i32p, f32p, i32p, i32p]
    L.ref_evalloader_run.restype = C.c_int
    L.ref_learning_rates.argtypes = [C.c_char_p, C.c_float, C.c_int, C.c_int, C.c_float, C.c_int, f32p]
    L.ref_tokenizer_decode.argtypes = [C.c_char_p, u32p, C.c_int, C.c_char_p, C.c_size_t, C.POINTER(C.c_uint)]
    L.ref_tokenizer_decode.restype = C.c_int
    f64p = np.ctypeslib.ndpointer(dtype=np.float64, flags="C_CONTIGUOUS")
    L.ref_detector_run.argtypes = [f64p, C.c_int, f64p]
    L.ref_logger_run.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_int, f32p]
    L.ref_num_threads.restype = C.c_int
    _ref = L
    return L


# ------------------------------------------------------------------------------------------
# convenience wrappers

def param_sizes(cfg):
    sz = np.zeros(16, dtype=np.uint64)
    tot = cref().cref_param_sizes(sz, C.byref(cfg))
    return [int(x) for x in sz], int(tot)


def init_params(cfg, seed=42):
    _, tot = param_sizes(cfg)
    p = np.zeros(tot, dtype=np.float32)
    cref().cref_init_params(p, C.byref(cfg), seed)
    return p


def make_tokens(B, T, V, seed):
    """uint16-range tokens uniform in [0, V); targets are the inputs shifted by one."""
    rng = np.random.RandomState(seed)
    stream = rng.randint(0, V, size=B * T + 1).astype(np.int32)
    return np.ascontiguousarray(stream[:-1]), np.ascontiguousarray(stream[1:])


def cref_train(cfg, params, inputs, targets, B, T, steps, lr=1e-4, b1=0.9, b2=0.999, eps=1e-8, wd=0.0,
               grad_clip=0.0, wd_mask_2d=0, grad_step=0, want_logits=False):
    """Returns dict(losses, grads, logits, step_ms, gradnorm, params) from the CPU restatement."""
    _, tot = param_sizes(cfg)
    p = params.copy()
    losses = np.zeros(steps, dtype=np.float32)
    grads = np.zeros(tot, dtype=np.float32)
    ms = np.zeros(steps, dtype=np.float32)
    gn = np.zeros(steps, dtype=np.float32)
    logits = np.zeros(B * T * cfg.padded_vocab_size, dtype=np.float32) if want_logits else None
    rc = cref().cref_gpt2_train(C.byref(cfg), p, inputs, targets, B, T, steps, lr, b1, b2, eps, wd, grad_clip,
                                wd_mask_2d, losses, _opt(grads), grad_step, _opt(logits), _opt(ms), _opt(gn))
    assert rc == 0
    return dict(losses=losses, grads=grads, logits=logits, step_ms=ms, gradnorm=gn, params=p)


def ref_train(ckpt_path, cfg, inputs, targets, B, T, steps, lr=1e-4, b1=0.9, b2=0.999, eps=1e-8, wd=0.0,
              grad_step=0, want_logits=False):
    """Same outputs from the compiled reference trainer (needs oracle/_ref)."""
    _, tot = param_sizes(cfg)
    losses = np.zeros(steps, dtype=np.float32)
    grads = np.zeros(tot, dtype=np.float32)
    ms = np.zeros(steps, dtype=np.float32)
    pout = np.zeros(tot, dtype=np.float32)
    logits = np.zeros(B * T * cfg.padded_vocab_size, dtype=np.float32) if want_logits else None
    rc = ref().ref_gpt2_train(ckpt_path.encode(), inputs.copy(), targets.copy(), B, T, steps, lr, b1, b2, eps, wd,
                              losses, _opt(grads), grad_step, _opt(logits), _opt(ms), _opt(pout))
    assert rc == 0
    return dict(losses=losses, grads=grads, logits=logits, step_ms=ms, params=pout)


def cref_generate(cfg, params, T, genT, eot_token, rng_seed=1337):
    """Tokens of the CPU restatement's generation loop (positions >= genT stay eot_token)."""
    tokens = np.zeros(T, dtype=np.int32)
    state = C.c_uint64(rng_seed)
    assert cref().cref_gpt2_generate(C.byref(cfg), params, tokens, T, genT, eot_token, C.byref(state)) == 0
    return tokens, state.value


def ref_generate(ckpt_path, T, genT, eot_token, rng_seed=1337):
    """The same loop run by the compiled reference (its CPU forward pass + llmc/sampler.h)."""
    tokens = np.zeros(T, dtype=np.int32)
    state = C.c_uint64(rng_seed)
    assert ref().ref_gpt2_generate(ckpt_path.encode(), tokens, T, genT, eot_token, C.byref(state)) == 0
    return tokens, state.value


def to_bf16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros(x.size, dtype=np.uint16)
    cref().cref_f32_to_bf16_array(out, x.reshape(-1), x.size)
    return out.reshape(x.shape)


def from_bf16_bits(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.zeros(h.size, dtype=np.float32)
    cref().cref_bf16_to_f32_array(out, h.reshape(-1), h.size)
    return out.reshape(h.shape)
