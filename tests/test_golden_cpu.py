"""The CPU restatement against the committed output of the reference's own trainer
(tests/golden/tiny_gpt2.npz, written by tests/golden/make_golden.py). Needs no GPU and no reference."""
import os

import numpy as np

import oracle_lib as ol

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_gpt2.npz")


def load_golden():
    g = np.load(GOLD)
    cfg = ol.Config(*[int(x) for x in g["config"]])
    return g, cfg


def test_oracle_reproduces_reference_fixture():
    g, cfg = load_golden()
    B, T, steps = int(g["B"]), int(g["T"]), int(g["steps"])
    params = ol.init_params(cfg, int(g["seed"]))
    # the seeded init is part of the fixture: same parameter stream as the reference run
    assert abs(params.astype(np.float64).sum() - float(g["param_checksum"])) < 1e-6
    assert abs(np.abs(params).astype(np.float64).sum() - float(g["param_abs_sum"])) < 1e-5
    lr, b1, b2, eps, wd = [float(x) for x in g["hyper"]]
    r = ol.cref_train(cfg, params, g["inputs"], g["targets"], B, T, steps, lr=lr, b1=b1, b2=b2, eps=eps, wd=wd,
                      grad_step=0, want_logits=True)
    np.testing.assert_allclose(r["losses"], g["losses"], rtol=3e-6)
    np.testing.assert_allclose(r["logits"][g["logits_idx"]], g["logits_val"], rtol=1e-4, atol=1e-5)
    scale = np.abs(g["grad_val_step0"]).max()
    assert np.abs(r["grads"][g["grad_idx"]] - g["grad_val_step0"]).max() <= 1e-5 * scale
    sizes, _ = ol.param_sizes(cfg)
    offs = np.cumsum([0] + sizes)
    norms = np.array([np.sqrt((r["grads"][offs[i]:offs[i + 1]].astype(np.float64) ** 2).sum()) for i in range(16)])
    np.testing.assert_allclose(norms, g["grad_norms_step0"], rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(r["params"][g["grad_idx"]], g["final_param_val"], rtol=1e-4, atol=2e-4)
    r3 = ol.cref_train(cfg, params, g["inputs"], g["targets"], B, T, 4, lr=lr, b1=b1, b2=b2, eps=eps, wd=wd, grad_step=3)
    scale3 = np.abs(g["grad_val_step3"]).max()
    assert np.abs(r3["grads"][g["grad_idx"]] - g["grad_val_step3"]).max() <= 2e-4 * scale3


def test_oracle_reproduces_reference_generation_fixture():
    g = np.load(os.path.join(os.path.dirname(GOLD), "tiny_gpt2_generate.npz"))
    cfg = ol.Config(*[int(x) for x in g["config"]])
    params = np.ascontiguousarray(ol.init_params(cfg, int(g["seed"])) * np.float32(g["param_scale"]), np.float32)
    tokens, state = ol.cref_generate(cfg, params, cfg.max_seq_len, int(g["genT"]), int(g["eot_token"]), int(g["rng_seed"]))
    np.testing.assert_array_equal(tokens, g["tokens"])
    assert state == int(g["rng_state_after"])
