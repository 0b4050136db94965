"""A pool larger than its device tier (/root/reference src/ops/cuda/experts.rs:34-62, ops/placement.rs:113-128): the
experts that do not fit device memory live in pinned host memory that the device addresses directly, every pooled tensor
is read through a table of per-expert addresses, and replace_experts_by_counts exchanges busy host experts with idle
device ones.  Where an expert lies must never change a value: every run here is compared bit for bit with the same run
on a backend that holds the whole pool in device memory (the reference's acceptance test,
the_35b_generates_identically_with_the_expert_pool_oversubscribed)."""
import numpy as np
import pytest

from util import nvfp4_weights, q8_0_weights, rng

pytestmark = pytest.mark.gpu


def prompt_ids(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).astype(np.uint32)


def run_model(gguf, exact, slots, batches, n_new, seed, fuse=False):
    """Prefill in the given batch sizes (so that every batch kernel reads through the tables), then greedy decode.
    Fusion is off on both sides: a tabled pool is read by the unfused kernels, and in fast mode those differ from the
    fused ones in summation order."""
    import inferred_hip as ih
    be = ih.Hip(exact=exact, fuse=fuse)
    if slots is not None:
        be.set_expert_slots(slots)
    hm = ih.Model(gguf); he = ih.Engine(hm, be, 512, max_batch=256)
    ids = prompt_ids(sum(batches), hm.n_vocab, seed)
    logits, at = [], 0
    for b in batches:
        logits.append(np.array(he.forward(ids[at:at + b])))
        at += b
    out = he.decode_greedy(n_new)
    moved = be.replace_experts_by_counts()
    out2 = he.decode_greedy(n_new)
    st, tc = be.expert_stats(), be.tier_counters()
    report = be.config_report()
    graph = be.graph_stats()
    err = be.take_error()
    he.close(); hm.close(); be.close()
    assert err is None, err
    return logits, np.array(out), np.array(out2), moved, st, tc, report, graph


@pytest.mark.parametrize("exact", [True, False])
def test_mid_model_is_identical_with_two_thirds_of_the_pool_in_host_memory(mid_gguf, exact):
    """NVFP4 experts at config 5's layer shape, 4 layers x 3 tensors x 32 experts = 384 entries, 130 device slots.
    Batches of 3 (one GEMV per pair), 48 (16-pair f16 tiles in fast mode, int8 tiles in exact mode) and 100 tokens
    (128-pair f16 tiles), then decode token by token, an exchange by counts, and more decode."""
    batches, n_new = [3, 48, 100], 12
    ref = run_model(mid_gguf, exact, None, batches, n_new, 11)
    two = run_model(mid_gguf, exact, 130, batches, n_new, 11)
    for a, b in zip(ref[0], two[0]):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(ref[1], two[1]) and np.array_equal(ref[2], two[2])
    st, tc = two[4], two[5]
    assert st.oversubscribed == 0 and st.slots == 130 and st.resident == 130 and st.host_slots == 384 - 130
    assert st.pool == 384 and st.fetched == 0
    assert st.lookups == ref[4].lookups                     # the same reads, wherever they were served from
    assert 0 < st.hits < st.lookups and tc.host_reads == st.lookups - st.hits
    # busy host experts changed places with idle device ones: by themselves at the pass boundaries (every 64 tokens of
    # evidence, a bounded number) and then to completion by the explicit call
    assert st.evictions > two[3] > 0
    assert ref[3] == 0 and ref[4].oversubscribed == 0 and ref[4].host_slots == 0
    assert "pinned host" in two[6] and "all-resident" in ref[6]
    if exact:
        # with fusion and the decode graph on, the routed FFN of a tabled pool stays unfused inside the captured graph:
        # still the same bits (exact mode's fused and unfused kernels agree), replayed after the exchange as well
        fused = run_model(mid_gguf, True, 130, batches, n_new, 11, fuse=True)
        for a, b in zip(ref[0], fused[0]):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert np.array_equal(ref[1], fused[1]) and np.array_equal(ref[2], fused[2])
        assert fused[7]["replays"] >= 2 * n_new - 6 and fused[4].evictions > 0


def test_tiny_q8_0_model_through_the_row_kernel_and_the_int8_tiles(tiny_gguf):
    """Q8_0 experts (16 experts top-4): batches of 10 tokens (2.5 pairs per expert: the row kernel in fast mode) and of
    40 (the int8 tiles), with a third of the 192 entries in device memory."""
    for exact in (False, True):
        ref = run_model(tiny_gguf, exact, None, [10, 40, 2], 8, 5)
        two = run_model(tiny_gguf, exact, 64, [10, 40, 2], 8, 5)
        for a, b in zip(ref[0], two[0]):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert np.array_equal(ref[1], two[1]) and np.array_equal(ref[2], two[2])
        assert two[4].host_slots == 192 - 64 and two[4].evictions > 0


def test_exchange_by_counts_moves_the_busy_experts_in():
    """One tensor of 12 experts, 4 device slots.  Reads go to experts 8..11 only: after replace_experts_by_counts those
    four sit in device memory (the next reads are all hits), the counts are kept, and a second call moves nothing."""
    import inferred_hip as ih
    from oracle import binding as ob
    orc = ob.Oracle(threads=1)
    r = rng(9)
    n_in, n_out, n_expert, n_used, n_tok = 64, 32, 12, 2, 6
    wb = q8_0_weights(orc, r, n_expert * n_out, n_in, std=1.0)
    ids = np.array([8, 9, 10, 11, 8, 10, 9, 11, 8, 9, 10, 11], np.uint32)
    x = r.standard_normal(n_tok * n_in).astype(np.float32)
    want = np.zeros(n_tok * n_used * n_out, np.float32)
    orc.matmul_experts(ob.experts(wb, ih.Q8_0, n_in, n_out, n_expert), ids, n_used, x, want)
    be = ih.Hip(exact=True)
    be.set_expert_slots(4)
    E = ih.experts(wb, ih.Q8_0, n_in, n_out, n_expert)
    route = ih.Hip.host_route(ids, None, n_used)

    def once():
        out = np.zeros_like(want)
        be.begin_pass(n_tok)
        be.matmul_experts(E, route, x, out)
        be.end_pass(); be.host_needs(out)
        assert be.take_error() is None
        return out

    assert np.array_equal(once().view(np.uint32), want.view(np.uint32))
    st = be.expert_stats()
    assert st.host_slots == 8 and st.hits == 0 and st.lookups == ids.size       # every read crossed the bus
    assert be.replace_experts_by_counts() == 4
    assert np.array_equal(once().view(np.uint32), want.view(np.uint32))
    st = be.expert_stats()
    assert st.hits == ids.size and st.lookups == 2 * ids.size and st.evictions == 4
    assert np.array_equal(be.expert_counts(wb, n_expert), 2 * np.bincount(ids, minlength=n_expert))
    assert be.replace_experts_by_counts() == 0
    frac, total = be.expert_coverage()
    assert total == 2 * ids.size and frac == 1.0      # the four busiest entries take every read
    be.close()
