"""Writes tests/golden/tiny_gpt2.npz: what the reference's own CPU trainer (train_gpt2.c, compiled
unmodified into oracle/_ref by oracle/Makefile) produces on a tiny seeded GPT-2,
tests/golden/tiny_gpt2_generate.npz: the tokens its forward pass and llmc/sampler.h generate from that model, and
tests/golden/data_path.npz: the batches its data loaders (llmc/dataloader.h) serve from seeded synthetic files and the
rates its schedules (llmc/schedulers.h) give.

Run in the build container, where the reference checkout exists:
    make -C oracle all _ref && python tests/golden/make_golden.py [train|generate|data]
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


def write_data_fixture():
    import data_files as df
    R = ol.ref()
    sizes, vocab, shard_seed = [1000, 777, 1301], 50257, 11
    B, T, rank, nproc, nb = 2, 8, 1, 2, 120
    out = dict(shard_sizes=np.array(sizes), vocab=vocab, shard_seed=shard_seed, B=B, T=T, rank=rank, nproc=nproc, nbatches=nb)
    with tempfile.TemporaryDirectory() as d:
        pattern, _ = df.synthetic_shards(d, sizes, vocab, shard_seed)
        for shuffle in (0, 1):
            inp = np.zeros((nb, B * T), np.int32); tgt = np.zeros_like(inp)
            si = np.zeros(nb, np.uint64); sa = np.zeros(nb, np.uint64)
            ntok = C.c_size_t(0)
            buf = C.create_string_buffer(1 << 16)
            n = R.ref_dataloader_run(pattern.encode(), B, T, rank, nproc, shuffle, nb, 0, inp.reshape(-1), tgt.reshape(-1),
                                     si, sa, C.byref(ntok), buf)
            out[f"inputs_shuffle{shuffle}"], out[f"targets_shuffle{shuffle}"] = inp, tgt
            out[f"pos_shuffle{shuffle}"] = np.stack([si, sa], 1)
            if shuffle:
                state = bytearray(buf.raw[:n])
                cut = n - (8 + 4 + 4 + 624 * 4 + 8)
                state[cut:cut + 8] = bytes(8)          # the generator's first field is never set by the reference
                out["state_shuffle1"] = np.frombuffer(bytes(state), np.uint8)
        eN, eseed, eB, eT, enb, lseed = 23, 12, 12, 40, 9, 13
        path = os.path.join(d, "eval.bin")
        df.write_eval_file(path, df.synthetic_eval_examples(eN, vocab, eseed))
        losses = np.random.RandomState(lseed).rand(enb, eB * eT).astype(np.float32)
        inp = np.zeros((enb, eB * eT), np.int32); tgt = np.zeros_like(inp)
        mask = np.zeros((enb, eB * eT), np.int8); label = np.zeros((enb, eB // 4), np.int32)
        correct = np.zeros(enb, np.int32); info = np.zeros(5, np.int32)
        R.ref_evalloader_run(path.encode(), eB, eT, 0, 1, enb, inp.reshape(-1), tgt.reshape(-1), mask.reshape(-1),
                             label.reshape(-1), losses.reshape(-1), correct, info)
        out.update(eval_examples=eN, eval_seed=eseed, eval_B=eB, eval_T=eT, eval_nbatches=enb, eval_loss_seed=lseed,
                   eval_inputs=inp, eval_targets=tgt, eval_mask=mask, eval_correct=correct)
    for kind in ("cosine", "linear", "constant", "wsd"):
        lrs = np.zeros(301, np.float32)
        R.ref_learning_rates(kind.encode(), 6e-4, 20, 300, 0.1, 301, lrs)
        out[f"lr_{kind}"] = lrs
    np.savez_compressed(os.path.join(HERE, "data_path.npz"), **out)
    print("data fixture: correct per eval batch", correct)


def main():
    assert ol.have_ref(), "build oracle/_ref first (needs the reference checkout)"
    which = sys.argv[1] if len(sys.argv) > 1 else "all"
    if which in ("generate", "all"):
        write_generate_fixture()
    if which in ("data", "all"):
        write_data_fixture()
    if which in ("generate", "data"):
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
