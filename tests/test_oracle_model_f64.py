"""The oracle's MODEL LOOP against an independent float64 restatement of the architecture (tests/f64_model.py).

The per-op tests pin each `orc_*` function; this one pins the order in which oracle/model.cpp strings them together
(layer kinds, residuals, q/gate split, norm before rope, cache write before attending, routing over all experts,
the per-expert and shared-expert second scales around the silu, the sigmoid gate of the shared expert, the final
norm, head and output scale), on a hand-sized all-F32 model whose GGUF file is written by the test's own writer:
a batched prefill and three decode steps, logits every time, recurrent state, conv window and KV rows at the end.
"""
import numpy as np
import pytest

import f64_model as fm
from oracle import binding as ob

PROMPT = [3, 17, 9, 9, 22]
DECODE = [5, 0, 13]
TOL = 2e-5          # of the largest logit / state entry: f32 rounding through two layers sits near 1e-6


@pytest.fixture(scope="module")
def hand_model(tmp_path_factory):
    W = fm.draw_weights(seed=7)
    path = tmp_path_factory.mktemp("f64") / "hand_f32.gguf"
    fm.write_model(path, W)
    return W, path


def oracle_run(path):
    m = ob.Model(path); e = ob.Engine(m, 16)
    logits = [e.forward(PROMPT)] + [e.forward([t]) for t in DECODE]
    state = dict(ssm=e.ssm_state(0), conv=e.conv_state(0), k=e.k_slab(0), v=e.v_slab(0))
    e.close(); m.close()
    return logits, state


def f64_run(W, mistake=None):
    f = fm.F64Model(W, 16, mistake)
    logits = []
    for i, t in enumerate(PROMPT + DECODE):
        lg, _ = f.token(t)
        if i >= len(PROMPT) - 1:
            logits.append(lg)
    return logits, f


def rel(a, b):
    return np.abs(np.asarray(a, np.float64) - b).max() / np.abs(b).max()


def test_oracle_loop_matches_the_float64_restatement(hand_model):
    W, path = hand_model
    got, state = oracle_run(path)
    want, f = f64_run(W)
    assert len(got) == len(want) == 1 + len(DECODE)
    for i, (a, b) in enumerate(zip(got, want)):
        assert np.isfinite(a).all()
        assert rel(a, b) < TOL, (i, rel(a, b))
        assert int(np.argmax(a)) == int(np.argmax(b))
    S = fm.Shape
    assert rel(state["ssm"].reshape(S.dt_rank, S.d_state, S.d_state), f.ssm) < TOL
    assert rel(state["conv"].reshape(S.conv_dim, S.d_conv - 1), f.conv_state) < TOL
    n = len(PROMPT) + len(DECODE)
    k = state["k"].view(np.float16).astype(np.float64).reshape(16, S.kv_dim)
    v = state["v"].view(np.float16).astype(np.float64).reshape(16, S.kv_dim)
    assert rel(k[:n], f.K[:n]) < 2e-3 and rel(v[:n], f.V[:n]) < 2e-3   # one f16 step where f32 and f64 round apart
    assert not k[n:].any() and not v[n:].any()


@pytest.mark.parametrize("mistake", fm.MISTAKES)
def test_the_comparison_tells_a_wrong_order_from_the_right_one(hand_model, mistake):
    """Each plausible slip, made on purpose in the float64 model, moves its logits off the oracle's by at least a
    hundred times the tolerance of the test above: the agreement there is not an accident of loose bounds."""
    W, path = hand_model
    got, _ = oracle_run(path)
    wrong, _ = f64_run(W, mistake)
    assert max(rel(a, b) for a, b in zip(got, wrong)) > 100 * TOL, mistake
