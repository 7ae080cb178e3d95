"""The host-side data path of the C-ABI library (include/llmk_data.h): shard loader, evaluation loader, learning-rate
schedules and token decoder, against the compiled reference (llmc/dataloader.h, schedulers.h, tokenizer.h through
oracle/_ref) where it is built, against the committed fixture everywhere, and against what the formats themselves fix.
All integer and byte work: bit-exact. No GPU is used (the library loads without one)."""
import ctypes as C
import os

import numpy as np
import pytest

import data_files as df
import gpu_lib
import oracle_lib as ol

needs_ref = pytest.mark.skipif(not ol.have_ref(), reason="oracle/_ref not built (needs the reference checkout)")
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "data_path.npz")

SHARD_SIZES = [1000, 777, 1301]
VOCAB = 50257


@pytest.fixture(scope="module")
def L():
    return gpu_lib.package().load("bf16")


class Loader:
    def __init__(self, L, pattern, B, T, rank=0, nproc=1, shuffle=0):
        self.L, self.n = L, B * T
        self.h = L.dataloader_create()
        L.dataloader_init(self.h, pattern.encode(), B, T, rank, nproc, shuffle)

    def next(self):
        self.L.dataloader_next_batch(self.h)
        return self.batch()

    def batch(self):
        inp = np.ctypeslib.as_array(self.L.dataloader_inputs(self.h), shape=(self.n,)).copy()
        tgt = np.ctypeslib.as_array(self.L.dataloader_targets(self.h), shape=(self.n,)).copy()
        return inp, tgt

    def pos(self):
        return self.L.dataloader_current_shard_idx(self.h), self.L.dataloader_current_sample_idx(self.h)

    def state(self):
        n = self.L.dataloader_get_shuffle_state(self.h, None)
        buf = C.create_string_buffer(n)
        assert self.L.dataloader_get_shuffle_state(self.h, buf) == n
        return buf.raw

    def free(self):
        self.L.dataloader_free(self.h)


def run_ours(L, pattern, B, T, rank, nproc, shuffle, nbatches, reset_every=0):
    ld = Loader(L, pattern, B, T, rank, nproc, shuffle)
    inp = np.zeros((nbatches, B * T), np.int32); tgt = np.zeros_like(inp)
    pos = np.zeros((nbatches, 2), np.uint64)
    for i in range(nbatches):
        if reset_every > 0 and i > 0 and i % reset_every == 0:
            L.dataloader_reset(ld.h)
        inp[i], tgt[i] = ld.next()
        pos[i] = ld.pos()
    ntok = L.dataloader_num_tokens(ld.h)
    state = ld.state() if shuffle else b""
    ld.free()
    return inp, tgt, pos, ntok, state


def run_ref(pattern, B, T, rank, nproc, shuffle, nbatches, reset_every=0):
    inp = np.zeros((nbatches, B * T), np.int32); tgt = np.zeros_like(inp)
    si = np.zeros(nbatches, np.uint64); sa = np.zeros(nbatches, np.uint64)
    ntok = C.c_size_t(0)
    buf = C.create_string_buffer(1 << 16)
    n = ol.ref().ref_dataloader_run(pattern.encode(), B, T, rank, nproc, shuffle, nbatches, reset_every, inp.reshape(-1),
                                    tgt.reshape(-1), si, sa, C.byref(ntok), buf)
    return inp, tgt, np.stack([si, sa], 1), ntok.value, buf.raw[:n]


# the generator state inside the shuffle state: 8 bytes the reference never sets, then left_, next_, words, MATRIX_A
RNG_BYTES = 8 + 4 + 4 + 624 * 4 + 8


def same_state(a, b):
    assert len(a) == len(b)
    cut = len(a) - RNG_BYTES
    assert a[:cut] == b[:cut] and a[cut + 8:] == b[cut + 8:]


@needs_ref
@pytest.mark.parametrize("shuffle", [0, 1])
@pytest.mark.parametrize("rank,nproc", [(0, 1), (1, 2), (2, 3)])
@pytest.mark.parametrize("reset_every", [0, 7])
def test_dataloader_matches_compiled_reference(L, tmp_path, shuffle, rank, nproc, reset_every):
    pattern, _ = df.synthetic_shards(str(tmp_path), SHARD_SIZES, VOCAB, seed=1)
    B, T, nb = 2, 8, 150          # several epochs: the three shards hold 190 / nproc samples
    ours = run_ours(L, pattern, B, T, rank, nproc, shuffle, nb, reset_every)
    ref = run_ref(pattern, B, T, rank, nproc, shuffle, nb, reset_every)
    np.testing.assert_array_equal(ours[0], ref[0])
    np.testing.assert_array_equal(ours[1], ref[1])
    np.testing.assert_array_equal(ours[2], ref[2])
    assert ours[3] == ref[3] == sum(SHARD_SIZES)
    if shuffle:
        same_state(ours[4], ref[4])


def test_dataloader_without_shuffle_is_a_strided_walk(L, tmp_path):
    pattern, toks = df.synthetic_shards(str(tmp_path), SHARD_SIZES, VOCAB, seed=2)
    B, T, rank, nproc = 2, 8, 1, 2
    n = B * T
    ld = Loader(L, pattern, B, T, rank, nproc, 0)
    assert L.dataloader_num_shards(ld.h) == 3 and L.dataloader_num_tokens(ld.h) == sum(SHARD_SIZES)
    assert L.dataloader_should_shuffle(ld.h) == 0
    # samples of the current shard for this process group: (tokens - 1) // (processes * B * T), llmc/dataloader.h:96
    assert L.dataloader_shard_num_samples(ld.h) == (toks[0].size - 1) // (nproc * n)
    for epoch in range(2):
        for s, t in enumerate(toks):
            for k in range((t.size - 1) // (nproc * n)):
                inp, tgt = ld.next()
                o = k * nproc * n + rank * n
                np.testing.assert_array_equal(inp, t[o:o + n].astype(np.int32))
                np.testing.assert_array_equal(tgt, t[o + 1:o + n + 1].astype(np.int32))
                assert ld.pos() == (s, k + 1)
    # load_batch re-reads the sample the position points at without moving on
    L.dataloader_resume(ld.h, 1, 3)
    L.dataloader_load_batch(ld.h)
    o = 3 * nproc * n + rank * n
    np.testing.assert_array_equal(ld.batch()[0], toks[1][o:o + n].astype(np.int32))
    assert ld.pos() == (1, 3)
    ld.free()


def test_dataloader_shuffle_visits_every_sample_once_per_epoch(L, tmp_path):
    pattern, toks = df.synthetic_shards(str(tmp_path), SHARD_SIZES, VOCAB, seed=3)
    B, T = 2, 8
    n = B * T
    per_shard = [(t.size - 1) // n for t in toks]
    starts = {}                         # first 16 tokens of every sample -> (shard, sample); random tokens: unique
    for s, t in enumerate(toks):
        for k in range(per_shard[s]):
            starts[t[k * n:k * n + n].tobytes()] = (s, k)
    assert len(starts) == sum(per_shard)
    ld = Loader(L, pattern, B, T, 0, 1, 1)
    orders = []
    for epoch in range(3):
        seen = []
        for _ in range(sum(per_shard)):
            inp, tgt = ld.next()
            s, k = starts[inp.astype(np.uint16).tobytes()]
            np.testing.assert_array_equal(tgt, toks[s][k * n + 1:k * n + n + 1].astype(np.int32))
            seen.append((s, k))
        assert sorted(seen) == sorted(starts.values())           # a permutation of all samples
        shard_order = [s for i, (s, _) in enumerate(seen) if i == 0 or seen[i - 1][0] != s]
        assert sorted(shard_order) == [0, 1, 2]                  # ... shard by shard
        orders.append(seen)
    assert orders[0] != orders[1] and orders[1] != orders[2]
    ld.free()
    other = Loader(L, pattern, B, T, 0, 1, 1)                    # same seed, same files: same order
    assert [starts[other.next()[0].astype(np.uint16).tobytes()] for _ in range(20)] == orders[0][:20]
    other.free()


@pytest.mark.parametrize("after", [5, 62, 63, 130])
def test_dataloader_shuffle_state_round_trip(L, tmp_path, after):
    """What save_state / load_state do with the loader (train_gpt2.cu:1228-1247, :1289-1310): position + shuffle state
    written after `after` batches, read into a fresh loader, and both continue with the same batches."""
    pattern, _ = df.synthetic_shards(str(tmp_path), SHARD_SIZES, VOCAB, seed=4)
    B, T = 2, 8
    a = Loader(L, pattern, B, T, 0, 1, 1)
    for _ in range(after):
        a.next()
    state, (shard, sample) = a.state(), a.pos()
    b = Loader(L, pattern, B, T, 0, 1, 1)
    assert L.dataloader_set_shuffle_state(b.h, state, len(state)) == len(state)
    L.dataloader_resume(b.h, shard, sample)
    assert b.state() == state
    for _ in range(140):
        x, y = a.next(), b.next()
        np.testing.assert_array_equal(x[0], y[0])
        np.testing.assert_array_equal(x[1], y[1])
        assert a.pos() == b.pos()
    a.free(); b.free()


# ---- evaluation loader -----------------------------------------------------------------------------------------

def run_eval_ours(L, path, B, T, rank, nproc, nbatches, losses):
    h = L.evalloader_create()
    L.evalloader_init(h, path.encode(), B, T, rank, nproc)
    info = [L.evalloader_num_examples(h), L.evalloader_num_batches(h), L.evalloader_start_example_index(h),
            L.evalloader_end_example_index(h)]
    can_fit = B // 4
    inp = np.zeros((nbatches, B * T), np.int32); tgt = np.zeros_like(inp)
    mask = np.zeros((nbatches, B * T), np.int8); label = np.zeros((nbatches, can_fit), np.int32)
    correct = np.zeros(nbatches, np.int32)
    for i in range(nbatches):
        L.evalloader_next_batch(h)
        inp[i] = np.ctypeslib.as_array(L.evalloader_inputs(h), shape=(B * T,))
        tgt[i] = np.ctypeslib.as_array(L.evalloader_targets(h), shape=(B * T,))
        mask[i] = np.frombuffer(C.string_at(L.evalloader_mask(h), B * T), np.int8)
        label[i] = np.ctypeslib.as_array(L.evalloader_label(h), shape=(can_fit,))
        correct[i] = L.evalloader_stat_losses(h, losses[i].ctypes.data_as(C.c_void_p))
    info.append(L.evalloader_current_example_index(h))
    L.evalloader_free(h)
    return inp, tgt, mask, label, correct, info


@needs_ref
@pytest.mark.parametrize("rank,nproc", [(0, 1), (1, 2), (2, 3)])
def test_evalloader_matches_compiled_reference(L, tmp_path, rank, nproc):
    path = str(tmp_path / "eval.bin")
    df.write_eval_file(path, df.synthetic_eval_examples(23, VOCAB, seed=5))
    B, T = 12, 40
    per = -(-23 // nproc)
    nb = -(-per // (B // 4)) + 1                      # one batch past the end: it must come back empty
    losses = np.random.RandomState(6).rand(nb, B * T).astype(np.float32)
    ours = run_eval_ours(L, path, B, T, rank, nproc, nb, losses)
    inp = np.zeros((nb, B * T), np.int32); tgt = np.zeros_like(inp)
    mask = np.zeros((nb, B * T), np.int8); label = np.zeros((nb, B // 4), np.int32)
    correct = np.zeros(nb, np.int32); info = np.zeros(5, np.int32)
    ol.ref().ref_evalloader_run(path.encode(), B, T, rank, nproc, nb, inp.reshape(-1), tgt.reshape(-1), mask.reshape(-1),
                                label.reshape(-1), losses.reshape(-1), correct, info)
    np.testing.assert_array_equal(ours[2], mask)
    # inputs and targets are only defined where an example wrote them: the whole arrays still agree because both
    # sides start from zero and never clear
    np.testing.assert_array_equal(ours[0], inp)
    np.testing.assert_array_equal(ours[1], tgt)
    np.testing.assert_array_equal(ours[4], correct)
    assert ours[5] == info.tolist()
    filled = [min(B // 4, max(0, info[3] - info[2] - i * (B // 4))) for i in range(nb)]
    for i, f in enumerate(filled):                     # labels of slots that were filled in this batch
        np.testing.assert_array_equal(ours[3][i, :f], label[i, :f])


def test_evalloader_layout_and_scoring(L, tmp_path):
    examples = df.synthetic_eval_examples(5, VOCAB, seed=7)
    path = str(tmp_path / "eval.bin")
    df.write_eval_file(path, examples)
    B, T = 8, 40
    losses = np.random.RandomState(8).rand(3, B * T).astype(np.float32)
    inp, tgt, mask, label, correct, info = run_eval_ours(L, path, B, T, 0, 1, 3, losses)
    assert info == [5, 3, 0, 5, 5]
    for i in range(3):
        want_correct = 0
        for slot in range(2):
            e = i * 2 + slot
            if e >= 5:
                assert not mask[i].reshape(B, T)[slot * 4:slot * 4 + 4].any()
                continue
            lab, ctx, comps = examples[e]
            assert label[i, slot] == lab
            means = []
            for c, comp in enumerate(comps):
                row = slot * 4 + c
                r_in, r_tg, r_mk = (a[i].reshape(B, T)[row] for a in (inp, tgt, mask))
                np.testing.assert_array_equal(r_in[:len(ctx) + len(comp)], ctx + comp)
                want_mask = np.zeros(T, np.int8); want_mask[len(ctx) - 1:len(ctx) - 1 + len(comp)] = 1
                np.testing.assert_array_equal(r_mk, want_mask)
                np.testing.assert_array_equal(r_tg[want_mask == 1], comp)
                means.append(np.float32(losses[i].reshape(B, T)[row][want_mask == 1].astype(np.float64).mean()))
            want_correct += int(np.argmin(means)) == lab
        assert correct[i] == want_correct
    # evalloader_reset (llmc/dataloader.h:298) goes back to the process's first example: the first batch comes again
    h = L.evalloader_create()
    L.evalloader_init(h, path.encode(), B, T, 0, 1)
    L.evalloader_next_batch(h); L.evalloader_next_batch(h)
    assert L.evalloader_current_example_index(h) == 4
    L.evalloader_reset(h)
    assert L.evalloader_current_example_index(h) == 0
    L.evalloader_next_batch(h)
    again = np.ctypeslib.as_array(L.evalloader_inputs(h), shape=(B * T,)).reshape(B, T)
    np.testing.assert_array_equal(np.frombuffer(C.string_at(L.evalloader_mask(h), B * T), np.int8), mask[0])
    for slot in range(2):                                          # the tokens past a row's end are left as they were
        lab, ctx, comps = examples[slot]
        for c, comp in enumerate(comps):
            np.testing.assert_array_equal(again[slot * 4 + c][:len(ctx) + len(comp)], ctx + comp)
    L.evalloader_free(h)


# ---- learning-rate schedules -------------------------------------------------------------------------------------

def ours_lrs(L, kind, lr, warmup, nb, frac, steps):
    h = L.lr_scheduler_create()
    L.lr_scheduler_init(h, kind.encode(), lr, warmup, nb, frac)
    out = np.array([L.get_learning_rate(h, s) for s in range(steps)], np.float32)
    L.lr_scheduler_free(h)
    return out


@needs_ref
@pytest.mark.parametrize("kind", ["cosine", "linear", "constant", "wsd"])
@pytest.mark.parametrize("lr,warmup,nb,frac", [(6e-4, 700, 18865, 0.0), (3e-4, 10, 200, 0.1), (1e-3, 0, 50, 1.0)])
def test_lr_schedules_match_compiled_reference(L, kind, lr, warmup, nb, frac):
    want = np.zeros(nb + 1, np.float32)
    ol.ref().ref_learning_rates(kind.encode(), lr, warmup, nb, frac, nb + 1, want)
    got = ours_lrs(L, kind, lr, warmup, nb, frac, nb + 1)
    # same float expressions; the two compilers may fuse a multiply-add or evaluate cosf differently in the last
    # place, which near the end of a decay to zero (lr - ratio * lr) is a last place of lr, not of the result
    np.testing.assert_allclose(got, want, rtol=3e-7, atol=lr * 1.2e-7)


def test_lr_schedules_closed_forms(L):
    lr, warmup, nb, frac = np.float32(6e-4), 10, 100, np.float32(0.1)
    for kind in ("cosine", "linear", "wsd"):
        got = ours_lrs(L, kind, lr, warmup, nb, frac, nb + 1)
        np.testing.assert_allclose(got[:warmup], lr * np.arange(1, warmup + 1, dtype=np.float32) / warmup, rtol=2e-7)
        assert got[warmup] == lr or kind == "wsd"                       # decay starts from the full rate
        np.testing.assert_allclose(got[nb], lr * frac, rtol=1e-6)        # ... and ends at the final fraction
        assert (np.diff(got[warmup:]) <= 1e-12).all()
    steps = np.arange(warmup, nb + 1)
    ratio = (steps - warmup) / (nb - warmup)
    np.testing.assert_allclose(ours_lrs(L, "cosine", lr, warmup, nb, frac, nb + 1)[warmup:],
                               lr * frac + 0.5 * (1 + np.cos(np.pi * ratio)) * (lr - lr * frac), rtol=2e-6)
    np.testing.assert_allclose(ours_lrs(L, "linear", lr, warmup, nb, frac, nb + 1)[warmup:], lr - ratio * (lr - lr * frac), rtol=2e-6)
    wsd = ours_lrs(L, "wsd", lr, warmup, nb, frac, nb + 1)
    assert (wsd[warmup:80] == lr).all()
    np.testing.assert_allclose(wsd[80:], lr * frac + (1 - np.sqrt((np.arange(80, nb + 1) - 80) / 20)) * (lr - lr * frac), rtol=2e-6)
    assert (ours_lrs(L, "constant", lr, warmup, nb, frac, nb + 1) == lr).all()


# ---- token decoder -----------------------------------------------------------------------------------------------

def make_pieces(n, seed):
    rs = np.random.RandomState(seed)
    return [bytes(rs.randint(1, 256, rs.randint(1, 12)).astype(np.uint8)) for _ in range(n)]   # no zero bytes: C strings


def test_tokenizer_decodes_the_table(L, tmp_path):
    pieces = make_pieces(300, 9)
    path = str(tmp_path / "tok.bin")
    df.write_tokenizer(path, pieces, eot_token=299)
    h = L.tokenizer_create()
    L.tokenizer_init(h, path.encode())
    assert L.tokenizer_init_ok(h) == 1 and L.tokenizer_eot_token(h) == 299 and L.tokenizer_vocab_size(h) == 300
    for i in (0, 1, 57, 299):
        assert C.string_at(L.tokenizer_decode(h, i)) == pieces[i]
    assert L.tokenizer_decode(h, 300) is None                         # outside the vocabulary
    L.tokenizer_free(h)
    h = L.tokenizer_create()
    L.tokenizer_init(h, str(tmp_path / "missing.bin").encode())       # a missing file is a warning, not an error
    assert L.tokenizer_init_ok(h) == 0 and L.tokenizer_decode(h, 0) is None
    L.tokenizer_free(h)


@needs_ref
def test_tokenizer_matches_compiled_reference(L, tmp_path):
    pieces = make_pieces(300, 10)
    path = str(tmp_path / "tok.bin")
    df.write_tokenizer(path, pieces, eot_token=7)
    ids = np.arange(300, dtype=np.uint32)
    out = C.create_string_buffer(8192)
    vocab = C.c_uint(0)
    eot = ol.ref().ref_tokenizer_decode(path.encode(), ids, 300, out, 8192, C.byref(vocab))
    ref_pieces = out.raw.split(b"\0")[:300]
    h = L.tokenizer_create()
    L.tokenizer_init(h, path.encode())
    assert (L.tokenizer_eot_token(h), L.tokenizer_vocab_size(h)) == (eot, vocab.value) == (7, 300)
    assert [C.string_at(L.tokenizer_decode(h, int(i))) for i in ids] == ref_pieces == pieces
    L.tokenizer_free(h)


# ---- outlier detector and run log -----------------------------------------------------------------------------------

def ours_z(L, values):
    h = L.outlier_detector_create()
    out = np.array([L.update_detector(h, float(v)) for v in values])
    L.outlier_detector_free(h)
    return out


def test_outlier_detector_is_the_z_score_of_the_last_128(L):
    v = np.random.RandomState(14).randn(400) * 3 + 10
    v[300] = 80.0                                         # an outlier
    z = ours_z(L, v)
    assert np.isnan(z[:128]).all() and not np.isnan(z[128:]).any()
    for i in (128, 129, 255, 300, 399):
        w = v[i - 127:i + 1]                              # the window already holds the new value
        np.testing.assert_allclose(z[i], (v[i] - w.mean()) / w.std(), rtol=1e-9)
    assert z[300] > 8 and np.abs(np.delete(z[128:], 300 - 128)).max() < 5
    assert (ours_z(L, np.full(200, 2.5))[128:] == 0).all()        # no spread: zero, not a division by zero


@needs_ref
def test_outlier_detector_matches_compiled_reference(L):
    v = np.random.RandomState(15).rand(1000) * 4 + 1
    want = np.zeros(1000)
    ol.ref().ref_detector_run(v, 1000, want)
    got = ours_z(L, v)
    assert (np.isnan(got) == np.isnan(want)).all()
    np.testing.assert_allclose(got[128:], want[128:], rtol=1e-10)


def ours_log(L, directory, rank, resume, n, vals):
    h = L.logger_create()
    L.logger_init(h, directory.encode() if directory else None, rank, resume)
    for i in range(n):
        L.logger_log_train(h, i, *[float(x) for x in vals[4 * i:4 * i + 3]])
        if i % 3 == 0:
            L.logger_log_val(h, i, float(vals[4 * i + 3]))
        if i % 5 == 0:
            L.logger_log_eval(h, i, float(np.float32(vals[4 * i + 3]) * np.float32(0.01)))
    L.logger_free(h)


def test_logger_lines(L, tmp_path):
    vals = np.array([3.14159, 6e-4, 1.2345, 2.5] * 3, np.float32)
    ours_log(L, str(tmp_path), 0, 0, 3, vals)
    assert open(tmp_path / "main.log").read() == ("s:0 trl:3.1416 lr:0.000600 norm:1.23\ns:0 tel:2.5000\ns:0 eval:0.0250\n"
                                                 "s:1 trl:3.1416 lr:0.000600 norm:1.23\ns:2 trl:3.1416 lr:0.000600 norm:1.23\n")
    ours_log(L, str(tmp_path), 0, 1, 1, vals)             # resuming appends
    assert open(tmp_path / "main.log").read().count("\n") == 8
    ours_log(L, str(tmp_path), 1, 0, 1, vals)             # other processes do not write (and do not empty the file)
    assert open(tmp_path / "main.log").read().count("\n") == 8
    ours_log(L, str(tmp_path), 0, 0, 1, vals)             # a fresh run starts over
    assert open(tmp_path / "main.log").read().count("\n") == 3


@needs_ref
def test_logger_matches_compiled_reference(L, tmp_path):
    vals = (np.random.RandomState(16).rand(4 * 17) * 10).astype(np.float32)
    a, b = tmp_path / "a", tmp_path / "b"
    a.mkdir(); b.mkdir()
    for resume in (0, 1):
        ours_log(L, str(a), 0, resume, 17, vals)
        ol.ref().ref_logger_run(str(b).encode(), 0, resume, 17, vals)
        assert open(a / "main.log", "rb").read() == open(b / "main.log", "rb").read()


# ---- the committed fixture: what the compiled reference produced, for machines without it ---------------------------

def test_data_path_reproduces_reference_fixture(L, tmp_path):
    g = np.load(GOLD)
    sizes, seed = [int(x) for x in g["shard_sizes"]], int(g["shard_seed"])
    pattern, _ = df.synthetic_shards(str(tmp_path), sizes, int(g["vocab"]), seed)
    B, T, rank, nproc, nb = (int(g[k]) for k in ("B", "T", "rank", "nproc", "nbatches"))
    for shuffle in (0, 1):
        inp, tgt, pos, _, state = run_ours(L, pattern, B, T, rank, nproc, shuffle, nb)
        np.testing.assert_array_equal(inp, g[f"inputs_shuffle{shuffle}"])
        np.testing.assert_array_equal(tgt, g[f"targets_shuffle{shuffle}"])
        np.testing.assert_array_equal(pos, g[f"pos_shuffle{shuffle}"])
        if shuffle:
            same_state(state, g["state_shuffle1"].tobytes())
    path = str(tmp_path / "eval.bin")
    df.write_eval_file(path, df.synthetic_eval_examples(int(g["eval_examples"]), int(g["vocab"]), int(g["eval_seed"])))
    eB, eT, enb = int(g["eval_B"]), int(g["eval_T"]), int(g["eval_nbatches"])
    losses = np.random.RandomState(int(g["eval_loss_seed"])).rand(enb, eB * eT).astype(np.float32)
    ours = run_eval_ours(L, path, eB, eT, 0, 1, enb, losses)
    np.testing.assert_array_equal(ours[0], g["eval_inputs"])
    np.testing.assert_array_equal(ours[1], g["eval_targets"])
    np.testing.assert_array_equal(ours[2], g["eval_mask"])
    np.testing.assert_array_equal(ours[4], g["eval_correct"])
    for kind in ("cosine", "linear", "constant", "wsd"):
        np.testing.assert_allclose(ours_lrs(L, kind, 6e-4, 20, 300, 0.1, 301), g[f"lr_{kind}"], rtol=3e-7, atol=6e-4 * 1.2e-7)
