"""Writes tests/golden/tiny_gpt2.npz: what the reference's own CPU trainer (train_gpt2.c, compiled
unmodified into oracle/_ref by oracle/Makefile) produces on a tiny seeded GPT-2, and
tests/golden/tiny_gpt2_generate.npz: the tokens its forward pass and llmc/sampler.h generate from that model.

Run in the build container, where the reference checkout exists:
    make -C oracle all _ref && python tests/golden/make_golden.py [train|generate]
The fixture holds data only: the configuration, the tokens, the per-step losses, and samples of
the logits, gradients and updated parameters (indices + values), so that the oracle restatement
and the GPU path can be checked against the reference on machines that do not have it.
"""
import ctypes as C
import os
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as ol  # noqa: E402

CFG = dict(max_seq_len=32, vocab_size=100, padded_vocab_size=128, num_layers=2, num_heads=2, channels=128)
B, T, STEPS, SEED, TOKEN_SEED = 2, 32, 10, 42, 7
HYPER = dict(lr=1e-3, b1=0.9, b2=0.999, eps=1e-8, wd=0.0)


GEN = dict(genT=32, eot_token=99, rng_seed=1337, param_scale=8.0)   # scaled weights: distributions far from uniform


def write_generate_fixture():
    cfg = ol.Config(**CFG)
    params = np.ascontiguousarray(ol.init_params(cfg, SEED) * np.float32(GEN["param_scale"]), np.float32)
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "tiny.bin")
        assert ol.cref().cref_write_checkpoint_fp32(path.encode(), params, C.byref(cfg)) == 0
        tokens, state = ol.ref_generate(path, cfg.max_seq_len, GEN["genT"], GEN["eot_token"], GEN["rng_seed"])
    np.savez_compressed(
        os.path.join(HERE, "tiny_gpt2_generate.npz"),
        config=np.array([CFG[k] for k in ("max_seq_len", "vocab_size", "padded_vocab_size", "num_layers", "num_heads", "channels")], np.int32),
        seed=SEED, param_scale=np.float32(GEN["param_scale"]), genT=GEN["genT"], eot_token=GEN["eot_token"],
        rng_seed=np.uint64(GEN["rng_seed"]), rng_state_after=np.uint64(state), tokens=tokens)
    print("tokens", tokens)


def main():
    assert ol.have_ref(), "build oracle/_ref first (needs the reference checkout)"
    which = sys.argv[1] if len(sys.argv) > 1 else "both"
    if which in ("generate", "both"):
        write_generate_fixture()
    if which == "generate":
        return
    cfg = ol.Config(**CFG)
    params = ol.init_params(cfg, SEED)
    inp, tgt = ol.make_tokens(B, T, cfg.vocab_size, TOKEN_SEED)
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "tiny.bin")
        assert ol.cref().cref_write_checkpoint_fp32(path.encode(), params, C.byref(cfg)) == 0
        r = ol.ref_train(path, cfg, inp, tgt, B, T, STEPS, grad_step=0, want_logits=True, **HYPER)
        r3 = ol.ref_train(path, cfg, inp, tgt, B, T, 4, grad_step=3, **HYPER)
    sizes, tot = ol.param_sizes(cfg)
    rng = np.random.RandomState(123)
    offs = np.cumsum([0] + sizes)
    idx = np.concatenate([offs[i] + rng.randint(0, sizes[i], min(256, sizes[i])) for i in range(16)]).astype(np.int64)
    lidx = rng.randint(0, r["logits"].size, 2048).astype(np.int64)
    norms = np.array([np.sqrt((r["grads"][offs[i]:offs[i + 1]].astype(np.float64) ** 2).sum()) for i in range(16)])
    np.savez_compressed(
        os.path.join(HERE, "tiny_gpt2.npz"),
        config=np.array([CFG[k] for k in ("max_seq_len", "vocab_size", "padded_vocab_size", "num_layers", "num_heads", "channels")], np.int32),
        B=B, T=T, steps=STEPS, seed=SEED, inputs=inp, targets=tgt,
        hyper=np.array([HYPER[k] for k in ("lr", "b1", "b2", "eps", "wd")], np.float64),
        param_checksum=np.float64(params.astype(np.float64).sum()), param_abs_sum=np.float64(np.abs(params).astype(np.float64).sum()),
        losses=r["losses"], logits_idx=lidx, logits_val=r["logits"][lidx],
        grad_idx=idx, grad_val_step0=r["grads"][idx], grad_val_step3=r3["grads"][idx], grad_norms_step0=norms,
        final_param_val=r["params"][idx])
    print("losses", r["losses"])


if __name__ == "__main__":
    main()
