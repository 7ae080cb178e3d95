"""Writers for the reference's on-disk data formats, for tests: token shards (llmc/dataloader.h:61-97), multiple-choice
evaluation files (llmc/dataloader.h:252-268) and tokenizer tables (llmc/tokenizer.h:41-84). Test infrastructure only."""
import numpy as np


def write_shard(path, tokens):
    tokens = np.asarray(tokens, dtype=np.uint16)
    header = np.zeros(256, dtype=np.int32)
    header[0], header[1], header[2] = 20240520, 1, tokens.size
    with open(path, "wb") as f:
        f.write(header.tobytes())
        f.write(tokens.tobytes())


def encode_example(index, label, context, completions):
    body = [label, len(completions), len(context), *context]
    for c in completions:
        body += [len(c), *c]
    nbytes = 2 * (3 + len(body))
    assert nbytes < 65536
    return np.array([65535, nbytes, index, *body], dtype=np.uint16)


def write_eval_file(path, examples):
    """examples: list of (label, context tokens, [4 completions])"""
    streams = [encode_example(i, lab, ctx, comps) for i, (lab, ctx, comps) in enumerate(examples)]
    header = np.zeros(256, dtype=np.int32)
    header[0], header[1], header[2], header[3] = 20240522, 1, len(streams), max(2 * s.size for s in streams)
    with open(path, "wb") as f:
        f.write(header.tobytes())
        for s in streams:
            f.write(s.tobytes())


def write_tokenizer(path, pieces, eot_token, version=2):
    header = np.zeros(256, dtype=np.uint32)
    header[0], header[1], header[2] = 20240328, version, len(pieces)
    if version == 2:
        header[3] = eot_token
    with open(path, "wb") as f:
        f.write(header.tobytes())
        for p in pieces:
            assert 0 < len(p) < 256
            f.write(bytes([len(p)]))
            f.write(p)


def synthetic_shards(directory, sizes, vocab, seed, prefix="train"):
    """Seeded shards `<prefix>_000000.bin`, ...; returns (glob pattern, list of token arrays)."""
    import os
    rs = np.random.RandomState(seed)
    toks = []
    for i, n in enumerate(sizes):
        t = rs.randint(0, vocab, n).astype(np.uint16)
        write_shard(os.path.join(directory, f"{prefix}_{i:06d}.bin"), t)
        toks.append(t)
    return os.path.join(directory, f"{prefix}_*.bin"), toks


def synthetic_eval_examples(n, vocab, seed, max_ctx=20, max_comp=12):
    rs = np.random.RandomState(seed)
    out = []
    for _ in range(n):
        ctx = rs.randint(0, vocab, rs.randint(1, max_ctx + 1)).tolist()
        comps = [rs.randint(0, vocab, rs.randint(1, max_comp + 1)).tolist() for _ in range(4)]
        out.append((int(rs.randint(0, 4)), ctx, comps))
    return out
