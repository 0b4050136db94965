"""The expert cache API with every expert in device memory (/root/reference src/ops/cuda/ops/placement.rs:15-363,
src/ops/cuda/experts.rs:210-315, 424-438, 890-901): device-side read counters, slab sizing, refusals."""
import numpy as np
import pytest

from util import q8_0_weights, rng

pytestmark = pytest.mark.gpu


def prompt_ids(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).astype(np.uint32)


@pytest.mark.parametrize("exact", [False, True])
def test_counters_after_a_greedy_run(mid_gguf, exact):
    """Every (tensor, pick) read is counted on the device by the expert kernels: eager prefill, eager decode and the
    replayed fused graph.  tokens x layers x n_used x 3 tensors, all served from device memory."""
    import inferred_hip as ih
    be = ih.Hip(exact=exact)
    assert be.expert_coverage() is None                        # no pooled tensor seen yet
    hm = ih.Model(mid_gguf); he = ih.Engine(hm, be, 128)
    n_prompt, n_new = 24, 13
    he.generate(prompt_ids(n_prompt, 8192, 3), n_new)
    assert be.take_error() is None
    tokens = n_prompt + n_new - 1                               # the last id is picked, not fed
    layers, n_expert, n_used = hm.n_layer, hm.n_expert, hm.n_expert_used
    st = be.expert_stats()
    assert st.lookups == tokens * layers * n_used * 3
    assert st.hits == st.lookups and st.host_slots == 0 and st.evictions == 0 and st.fetched == 0
    assert st.resident == n_expert * 3 * layers and st.pool == n_expert * 3 * layers
    assert st.oversubscribed == 0 and st.slots >= st.resident
    assert st.slot_bytes == 512 * 2048 // 64 * 36               # one NVFP4 expert matrix of the file
    frac, total = be.expert_coverage()
    assert total == st.lookups and frac == 1.0                  # every read hit a resident expert
    assert be.replace_experts_by_counts() == 0                  # nothing on a slower tier to promote
    tc = be.tier_counters()
    assert tc.lookups == st.lookups and tc.host_reads == 0 and tc.oversubscribed == 0 and tc.slots == st.slots
    assert be.graph_stats()["replays"] >= 5                     # the fused graph took part in the count
    assert "expert tier=all-resident" in be.config_report()
    he.close(); hm.close(); be.close()


def test_per_expert_counts_follow_the_route():
    import inferred_hip as ih
    from oracle import binding as ob
    orc = ob.Oracle(threads=1)
    be = ih.Hip(exact=False)
    r = rng(3)
    n_in, n_out, n_expert, n_used, n_tok = 64, 64, 12, 3, 40
    wb = q8_0_weights(orc, r, n_expert * n_out, n_in, std=1.0)
    ids = np.stack([r.permutation(n_expert)[:n_used] for _ in range(n_tok)]).astype(np.uint32).reshape(-1)
    x = r.standard_normal(n_tok * n_in).astype(np.float32); out = np.zeros(n_tok * n_used * n_out, np.float32)
    be.begin_pass(n_tok)
    E = ih.experts(wb, ih.Q8_0, n_in, n_out, n_expert)
    route = ih.Hip.host_route(ids, None, n_used)
    be.matmul_experts(E, route, x, out)
    be.matmul_experts(E, route, x, out)
    be.end_pass()
    assert be.take_error() is None
    got = be.expert_counts(wb, n_expert)
    assert np.array_equal(got, 2 * np.bincount(ids, minlength=n_expert))
    assert be.expert_stats().lookups == 2 * ids.size
    be.close()


def test_refusals():
    import inferred_hip as ih
    from oracle import binding as ob
    orc = ob.Oracle(threads=1)
    r = rng(4)
    n_in, n_out, n_expert = 64, 32, 8
    wb = q8_0_weights(orc, r, n_expert * n_out, n_in, std=1.0)
    ids = np.zeros(2, np.uint32); x = np.zeros(n_in, np.float32)
    route = ih.Hip.host_route(ids, None, 2)
    # a tensor whose byte length is not n_expert matrices of its shape (experts.rs:1621-1630)
    be = ih.Hip()
    be.begin_pass(1)
    bad = ih.experts(wb[:-34], ih.Q8_0, n_in, n_out, n_expert)
    be.matmul_experts(bad, route, x, np.zeros(2 * n_out, np.float32))
    assert "not n_expert matrices" in (be.take_error() or "")
    # a second pooled tensor of another matrix size: the slab's slot is uniform (experts.rs:890-901)
    be.matmul_experts(ih.experts(wb, ih.Q8_0, n_in, n_out, n_expert), route, x, np.zeros(2 * n_out, np.float32))
    assert be.take_error() is None
    wb2 = q8_0_weights(orc, r, n_expert * 2 * n_out, n_in, std=1.0)
    be.matmul_experts(ih.experts(wb2, ih.Q8_0, n_in, 2 * n_out, n_expert), route, x, np.zeros(4 * n_out, np.float32))
    assert "not uniform" in (be.take_error() or "")
    be.end_pass(); be.close()
    # a slab fixed at fewer slots than the pool needs spills into the pinned host tier (tests/test_gpu_expert_tiers.py);
    # with that tier's budget used up as well the rest is cold and fetched when picked (tests/test_gpu_expert_cold.py)
    be = ih.Hip()
    be.set_expert_slots(n_expert - 1)
    be.set_expert_host_budget(1)
    be.begin_pass(1)
    be.matmul_experts(ih.experts(wb, ih.Q8_0, n_in, n_out, n_expert), route, x, np.zeros(2 * n_out, np.float32))
    be.end_pass()
    assert be.take_error() is None
    st = be.expert_stats()
    assert st.slots == 7 and st.resident == 7 and st.host_slots == 0 and st.oversubscribed == 1 and st.fetched == 0
    be.close()
    # a budget in bytes sizes the slab the same way: three slots, five experts in the host tier
    be = ih.Hip()
    be.set_expert_budget(3 * n_out * n_in // 32 * 34)
    be.begin_pass(1)
    be.matmul_experts(ih.experts(wb, ih.Q8_0, n_in, n_out, n_expert), route, x, np.zeros(2 * n_out, np.float32))
    be.end_pass()
    assert be.take_error() is None
    st = be.expert_stats()
    assert st.slots == 3 and st.resident == 3 and st.host_slots == 5 and st.oversubscribed == 0   # nothing is cold
    be.close()


def test_qwen4exp_only_methods_are_refused_not_run():
    """The trait methods only the qwen4exp architecture calls (src/ops/mod.rs:705-966) are exported, launch nothing
    and leave their name in the sticky error."""
    import inferred_hip as ih
    be = ih.Hip()
    L, h = be.L, be.h
    x = np.ones(8, np.float32); p = x.ctypes.data
    calls = [("mean_streams", lambda: L.it_hip_mean_streams(h, p, 8, 2, 4, 0.5, p, 4)),
             ("mul_rows", lambda: L.it_hip_mul_rows(h, p, 8, p, 4)), ("silu", lambda: L.it_hip_silu(h, p, 8)),
             ("sigmoid", lambda: L.it_hip_sigmoid(h, p, 8)),
             ("mul_streams", lambda: L.it_hip_mul_streams(h, p, 8, p, 4, p, 2, 2)),
             ("row_dot", lambda: L.it_hip_row_dot(h, p, 8, p, 8, 4, p, 2)),
             ("signed_sqrt_sigmoid", lambda: L.it_hip_signed_sqrt_sigmoid(h, p, 8)),
             ("dilated_conv", lambda: L.it_hip_dilated_conv(h, p, 4, p, 8, p, 8, 2, 1, p, 8)),
             ("qsa_pool", lambda: L.it_hip_qsa_pool(h, p, 8, p, 8, None)),
             ("qsa_select", lambda: L.it_hip_qsa_select(h, p, 8, p, 8, None, p, 8, p, 8)),
             ("attend_sparse", lambda: L.it_hip_attend_sparse(h, None, p, 8, None, p, 8))]
    before = be.launch_count()
    for name, call in calls:
        call()
        err = be.take_error() or ""
        assert err.startswith(name + ":") and "qwen4exp-only" in err, (name, err)
    assert be.launch_count() == before and np.array_equal(x, np.ones(8, np.float32))
    be.close()
