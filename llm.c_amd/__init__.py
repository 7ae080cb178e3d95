"""Python host side of the MI355X kernel library for llm.c's GPT-2 training step.

This module only binds the C ABI declared in include/llmk.h (kernel launchers, one per launcher of
the reference's llmc/*.cuh), include/llmk_gpt2.h (the host GPT-2 driver) and include/llmk_data.h (data loaders,
learning-rate schedules, token decoder) through ctypes. There is
no Python or CPU implementation of any operation here: if the shared library has not been built
(python llm.c_amd/build.py), loading raises.

The directory name contains a dot, so import it by path:

    import importlib.util, sys
    spec = importlib.util.spec_from_file_location("llmc_amd", "llm.c_amd/__init__.py")
    llmc_amd = importlib.util.module_from_spec(spec); sys.modules["llmc_amd"] = llmc_amd
    spec.loader.exec_module(llmc_amd)
    lib = llmc_amd.load("bf16")
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIBDIR = os.path.join(HERE, "lib")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")

vp = C.c_void_p
ip = C.POINTER(C.c_int)
fp = C.POINTER(C.c_float)
sz = C.c_size_t
pd = C.c_ssize_t
i32 = C.c_int
f32 = C.c_float
u32 = C.c_uint

# name -> (restype, argtypes). Order of arguments = order in the headers.
KERNEL_ABI = {
    "llmk_init": (None, [i32]),
    "llmk_shutdown": (None, []),
    "llmk_precision": (C.c_char_p, []),
    "llmk_sizeof_floatx": (i32, []),
    "llmk_device_props": (None, [ip, ip, C.c_char_p]),
    "llmk_set_error_mode": (None, [i32]),
    "llmk_last_error": (C.c_char_p, []),
    "llmk_clear_error": (None, []),
    "llmk_profile_enable": (None, [i32]),
    "llmk_matmul_backward_split_mode": (None, [i32]),
    "llmk_gelu_forward_keep_grad": (None, [vp, vp, i32, vp]),
    "llmk_gelu_backward_from_grad": (None, [vp, vp, i32, vp]),
    "llmk_matmul_backward_last_split": (None, [ip, ip]),
    "llmk_matmul_backward_workspace_bytes": (sz, [i32, i32, i32, i32]),
    "llmk_attention_backward_workspace_bytes": (sz, [i32, i32, i32]),
    "llmk_workspace_reserve": (None, [sz]),
    "llmk_workspace_bytes": (sz, []),
    "llmk_profile_only": (None, [C.c_char_p]),
    "llmk_zero": (None, [vp, C.c_size_t, vp]),
    "llmk_probe_mfma_peak": (None, [C.POINTER(C.c_double), vp, vp]),
    "llmk_profile_reset": (None, []),
    "llmk_profile_count": (i32, []),
    "llmk_profile_get": (None, [i32, C.c_char_p, ip, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "llmk_encoder_forward": (None, [vp, vp, vp, vp, i32, i32, i32, vp]),
    "llmk_encoder_backward": (None, [vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, u32, vp]),
    "llmk_layernorm_forward": (None, [vp, vp, vp, vp, vp, vp, i32, i32, i32, vp]),
    "llmk_residual_forward": (None, [vp, vp, vp, i32, vp]),
    "llmk_fused_residual_forward5": (None, [vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, vp]),
    "llmk_layernorm_backward": (None, [vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp]),
    "llmk_layernorm_backward_scratch_floats": (sz, [i32]),
    "llmk_matmul_forward": (None, [vp, vp, vp, vp, i32, i32, i32, i32, vp, vp, i32]),
    "llmk_matmul_forward_residual": (None, [vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]),
    "llmk_matmul_backward": (None, [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp, vp, i32]),
    "llmk_matmul_backward_bias_scratch_floats": (sz, [i32]),
    "llmk_gelu_backward_bias": (None, [vp, vp, vp, vp, i32, i32, i32, vp]),
    "llmk_attention_forward": (None, [vp, vp, vp, i32, i32, i32, i32, vp]),
    "llmk_attention_backward": (None, [vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]),
    "llmk_attention_forward_fallback": (None, [vp, vp, vp, vp, i32, i32, i32, i32, vp]),
    "llmk_attention_backward_fallback": (None, [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]),
    "llmk_attention_backward_static": (None, [vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]),
    "llmk_gelu_forward": (None, [vp, vp, i32, vp]),
    "llmk_gelu_backward_inplace": (None, [vp, vp, i32, vp]),
    "llmk_fused_classifier": (None, [vp, vp, f32, vp, i32, i32, i32, i32, i32, vp]),
    "llmk_get_max_num_block_sums": (i32, [ip, i32]),
    "llmk_global_norm_squared": (None, [vp, vp, sz, pd, i32, i32, i32, vp]),
    "llmk_global_sum_deterministic": (None, [vp, vp, i32, vp]),
    "llmk_adamw_update": (None, [vp, vp, vp, vp, vp, sz, pd, pd, pd, i32, f32, f32, f32, i32, f32, f32, f32, u32, vp]),
    "llmk_adamw_update_multi": (i32, [vp, vp, vp, vp, vp, i32, vp, vp, vp, vp, vp, C.c_float, C.c_float, C.c_float, i32,
                                      C.c_float, C.c_float, vp]),
    "llmk_adamw_update_multi_clip": (i32, [vp, vp, vp, vp, vp, i32, vp, vp, vp, vp, vp, C.c_float, C.c_float, C.c_float, i32,
                                           C.c_float, vp, C.c_float, vp]),
    "llmk_init_from_master": (None, [vp, vp, sz, pd, pd, i32, u32, vp]),
    "llmk_copy_and_cast_to_f32": (None, [vp, vp, sz, pd, pd, i32, vp]),
}

DRIVER_ABI = {
    "gpt2_create": (vp, []),
    "gpt2_set_options": (None, [vp, i32, i32, i32]),
    "gpt2_build_from_descriptor": (None, [vp, C.c_char_p]),
    "gpt2_build_from_config": (None, [vp, i32, i32, i32, i32, i32, i32, u32]),
    "gpt2_build_from_checkpoint": (None, [vp, C.c_char_p, i32]),
    "gpt2_write_to_checkpoint": (None, [vp, C.c_char_p]),
    "gpt2_allocate_state": (None, [vp, i32, i32]),
    "gpt2_forward": (None, [vp, vp, sz, sz]),
    "gpt2_validate": (f32, [vp, vp, vp, sz, sz]),
    "gpt2_generate": (None, [vp, vp, i32, i32, C.POINTER(C.c_ulonglong)]),
    "gpt2_backward_and_reduce": (None, [vp, vp, vp, i32, i32]),
    "gpt2_calculate_grad_norm": (f32, [vp]),
    "gpt2_update": (None, [vp, f32, f32, f32, f32, f32, f32, i32, i32]),
    "gpt2_train_step": (None, [vp, vp, vp, f32, f32, f32, f32, f32, f32, i32, vp, vp]),
    "gpt2_estimate_mfu": (f32, [vp, i32, f32]),
    "gpt2_free": (None, [vp]),
    "gpt2_save_state": (None, [vp, C.c_char_p, i32]),
    "gpt2_load_state": (None, [vp, C.c_char_p, ip]),
    "gpt2_save_state_with_loader": (None, [C.c_char_p, i32, vp, vp]),
    "gpt2_load_state_with_loader": (None, [ip, vp, vp, C.c_char_p]),
    "gpt2_mean_loss": (f32, [vp]),
    "gpt2_num_parameters": (sz, [vp]),
    "gpt2_get_config": (None, [vp, ip]),
    "gpt2_param_sizes": (None, [vp, C.POINTER(sz)]),
    "gpt2_cpu_losses": (fp, [vp]),
    "gpt2_params_memory": (vp, [vp]),
    "gpt2_grads_memory": (vp, [vp]),
    "gpt2_output_memory": (vp, [vp]),
    "gpt2_get_params_f32": (None, [vp, vp]),
    "gpt2_set_params_f32": (None, [vp, vp]),
    "gpt2_get_grads_f32": (None, [vp, vp]),
    "gpt2_get_logits_f32": (None, [vp, vp, sz, sz]),
    "gpt2_get_rng_state": (C.c_ulonglong, [vp]),
    "gpt2_set_rng_state": (None, [vp, C.c_ulonglong]),
    "gpt2_activation_bytes": (sz, [vp]),
}


# include/llmk_data.h: shard loader, evaluation loader, learning-rate schedules, token decoder (host only)
u64p = C.POINTER(C.c_size_t)
DATA_ABI = {
    "dataloader_create": (vp, []),
    "dataloader_init": (None, [vp, C.c_char_p, sz, sz, i32, i32, i32]),
    "dataloader_reset": (None, [vp]),
    "dataloader_load_batch": (None, [vp]),
    "dataloader_next_batch": (None, [vp]),
    "dataloader_resume": (None, [vp, sz, sz]),
    "dataloader_free": (None, [vp]),
    "dataloader_inputs": (ip, [vp]),
    "dataloader_targets": (ip, [vp]),
    "dataloader_num_tokens": (sz, [vp]),
    "dataloader_num_shards": (sz, [vp]),
    "dataloader_shard_num_samples": (sz, [vp]),
    "dataloader_current_shard_idx": (sz, [vp]),
    "dataloader_current_sample_idx": (sz, [vp]),
    "dataloader_should_shuffle": (i32, [vp]),
    "dataloader_get_shuffle_state": (sz, [vp, vp]),
    "dataloader_set_shuffle_state": (sz, [vp, vp, sz]),
    "evalloader_create": (vp, []),
    "evalloader_init": (None, [vp, C.c_char_p, sz, sz, i32, i32]),
    "evalloader_reset": (None, [vp]),
    "evalloader_next_batch": (None, [vp]),
    "evalloader_stat_losses": (i32, [vp, vp]),
    "evalloader_free": (None, [vp]),
    "evalloader_inputs": (ip, [vp]),
    "evalloader_targets": (ip, [vp]),
    "evalloader_mask": (C.POINTER(C.c_char), [vp]),
    "evalloader_label": (ip, [vp]),
    "evalloader_num_examples": (i32, [vp]),
    "evalloader_num_batches": (i32, [vp]),
    "evalloader_start_example_index": (i32, [vp]),
    "evalloader_end_example_index": (i32, [vp]),
    "evalloader_current_example_index": (i32, [vp]),
    "lr_scheduler_create": (vp, []),
    "lr_scheduler_init": (None, [vp, C.c_char_p, f32, i32, i32, f32]),
    "get_learning_rate": (f32, [vp, i32]),
    "lr_scheduler_free": (None, [vp]),
    "tokenizer_create": (vp, []),
    "tokenizer_init": (None, [vp, C.c_char_p]),
    "tokenizer_decode": (vp, [vp, u32]),          # char* kept as an address: NULL is a valid answer
    "safe_printf": (None, [C.c_char_p]),
    "tokenizer_free": (None, [vp]),
    "tokenizer_init_ok": (i32, [vp]),
    "tokenizer_eot_token": (i32, [vp]),
    "tokenizer_vocab_size": (u32, [vp]),
    "outlier_detector_create": (vp, []),
    "init_detector": (None, [vp]),
    "update_detector": (C.c_double, [vp, C.c_double]),
    "outlier_detector_free": (None, [vp]),
    "logger_create": (vp, []),
    "logger_init": (None, [vp, C.c_char_p, i32, i32]),
    "logger_log_eval": (None, [vp, i32, f32]),
    "logger_log_val": (None, [vp, i32, f32]),
    "logger_log_train": (None, [vp, i32, f32, f32, f32]),
    "logger_free": (None, [vp]),
}


def lib_path(precision):
    return os.path.join(LIBDIR, f"libllmk_{precision}.so")


class LibraryMissing(RuntimeError):
    pass


_loaded = {}


def bind(lib):
    """Types every entry point of an opened library (include/llmk.h, llmk_gpt2.h) and returns it."""
    for table in (KERNEL_ABI, DRIVER_ABI, DATA_ABI):
        for name, (res, args) in table.items():
            fn = getattr(lib, name)   # AttributeError here = header and library disagree
            fn.restype = res
            fn.argtypes = args
    return lib


def load(precision="bf16"):
    """Loads lib/libllmk_<precision>.so and types every entry point. Raises if it is not built."""
    if precision not in ("bf16", "fp32"):
        raise ValueError("precision must be 'bf16' or 'fp32'")
    if precision in _loaded:
        return _loaded[precision]
    path = lib_path(precision)
    if not os.path.exists(path):
        raise LibraryMissing(f"{path} not found: build it with `python llm.c_amd/build.py` "
                             "(there is no fallback implementation)")
    lib = bind(C.CDLL(path))
    got = lib.llmk_precision().decode()
    if got != precision:
        raise RuntimeError(f"{path} reports precision {got}")
    _loaded[precision] = lib
    return lib
