"""The whole per-token loop on the MI355X against the CPU oracle on the same GGUF.

Config 1 of the baseline: 32 random prompt ids, greedy decode of 64 tokens — the ids
must be bit-identical, and so must the logits, recurrent state and KV slabs.
Structural properties the reference asserts on real models (tests/qwen35.rs:93-140,
348-396; tests/kv_cache.rs:45-176) are re-asserted here on the synthetic one.
"""
import numpy as np
import pytest

from util import assert_bits_equal

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    import inferred_hip as ih
    be = ih.Hip(exact=True)
    yield be
    be.close()


def prompt_ids(n=32, vocab=4096, seed=0):
    return np.random.default_rng(seed).integers(0, vocab, n).astype(np.uint32)


@pytest.mark.parametrize("which", ["tiny_gguf", "tiny_nvfp4_gguf"])
def test_greedy_tokens_bit_identical(hip, request, which):
    import inferred_hip as ih
    from oracle import binding as ob
    path = request.getfixturevalue(which)
    hip.drop_mirrors()  # resident weights are keyed on mmap addresses; a new file may reuse them
    prompt = prompt_ids()
    om = ob.Model(path); oe = ob.Engine(om, 128)
    ids_o, logits_o = oe.generate(prompt, 64)
    hm = ih.Model(path); he = ih.Engine(hm, hip, 128)
    ids_h, logits_h = he.generate(prompt, 64)
    print("oracle:", ids_o[:16], "\nhip:   ", ids_h[:16])
    assert len(ids_h) == 64
    assert np.array_equal(ids_o, ids_h), f"first divergence at {np.flatnonzero(ids_o != ids_h)[:1]}"
    assert_bits_equal(logits_h, logits_o, "final logits")
    for layer in range(3):
        assert_bits_equal(he.ssm_state(layer), oe.ssm_state(layer), f"ssm state {layer}")
        assert_bits_equal(he.conv_state(layer), oe.conv_state(layer), f"conv state {layer}")
    assert np.array_equal(he.k_slab(0), oe.k_slab(0)) and np.array_equal(he.v_slab(0), oe.v_slab(0))
    he.close(); hm.close(); oe.close(); om.close()


def test_batched_prefill_equals_token_by_token(hip, tiny_gguf):
    import inferred_hip as ih
    hip.drop_mirrors()
    hm = ih.Model(tiny_gguf)
    prompt = prompt_ids(40, seed=3)
    e1 = ih.Engine(hm, hip, 64); l1 = e1.forward(prompt)
    e2 = ih.Engine(hm, hip, 64)
    for t in prompt:
        l2 = e2.forward([t])
    assert_bits_equal(l1, l2, "batched vs token-by-token logits")
    assert_bits_equal(e1.ssm_state(0), e2.ssm_state(0), "state")
    # split prefill == single prefill
    e3 = ih.Engine(hm, hip, 64, max_batch=16); l3 = e3.prefill(prompt)
    assert_bits_equal(l1, l3, "split prefill")
    # reset reproduces the run (forget_state re-uploads the zeroed slabs)
    e1.reset(); l4 = e1.forward(prompt)
    assert_bits_equal(l1, l4, "after reset")
    for e in (e1, e2, e3):
        e.close()
    hm.close()


def test_context_overflow_is_refused_before_any_write(hip, tiny_gguf):
    import inferred_hip as ih
    hip.drop_mirrors()
    hm = ih.Model(tiny_gguf); e = ih.Engine(hm, hip, 8)
    with pytest.raises(ih.HipError, match="context overflow"):
        e.forward(prompt_ids(9))
    assert e.pos == 0
    e.close(); hm.close()
