"""A pool larger than both of its tiers (/root/reference src/ops/cuda/experts.rs:67-93, 1047-1190, 1418-1540,
2112-2233): experts that found room neither in device memory nor in pinned host memory are cold.  Before an expert
kernel runs the picks are read back, each cold pick is fetched from the model file into a device slot taken from an
expert the layer did not pick (GCLOCK with leases), and the placement tables are patched.  Where an expert lies must
never change a value: every run here is compared bit for bit with the same run on a backend that holds the whole pool in
device memory (the reference's acceptance test, the_35b_generates_identically_with_the_expert_pool_oversubscribed,
tests/cuda_ops.rs:6475-6633)."""
import os

import numpy as np
import pytest

from util import q8_0_weights, rng

pytestmark = pytest.mark.gpu

MID_EXPERT_BYTES = 512 * 2048 // 2 + 512 * 2048 // 16   # one repacked NVFP4 expert matrix of the mid model


def prompt_ids(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).astype(np.uint32)


def run_model(gguf, exact, slots, host_experts, batches, n_new, seed, prefetch=True, expert_bytes=MID_EXPERT_BYTES, fuse=False):
    """Fusion is off unless asked for: in fast mode the fused single-token kernels sum in another order than the unfused
    ones, and the comparison here is bit for bit."""
    import inferred_hip as ih
    be = ih.Hip(exact=exact, fuse=fuse)
    if slots is not None:
        be.set_expert_slots(slots)
        be.set_expert_host_budget(max(1, host_experts * expert_bytes))
    be.set_prefetch(prefetch)
    hm = ih.Model(gguf); he = ih.Engine(hm, be, 512, max_batch=256)
    ids = prompt_ids(sum(batches), hm.n_vocab, seed)
    logits, at = [], 0
    for b in batches:
        logits.append(np.array(he.forward(ids[at:at + b])))
        at += b
    out = np.array(he.decode_greedy(n_new))
    moved = be.replace_experts_by_counts()
    st, tc = be.expert_stats(), be.tier_counters()
    report, graph = be.config_report(), be.graph_stats()
    run_model.reads = be.fetch_read_counts()
    err = be.take_error()
    he.close(); hm.close(); be.close()
    assert err is None, err
    return logits, out, st, tc, report, graph, moved


@pytest.mark.parametrize("exact", [True, False])
def test_mid_model_is_identical_with_cold_experts(mid_gguf, exact):
    """4 layers x 3 tensors x 32 experts = 384 entries; 130 device slots, 100 pinned blocks, 154 cold.  Batches of 3, 48
    and 100 tokens (a layer's batch picks every expert: 96 leased slots), then decode token by token (30 leased), with
    the bytes read from the model file by the reader threads and the lookahead on."""
    batches, n_new = [3, 48, 100], 16
    ref = run_model(mid_gguf, exact, None, 0, batches, n_new, 11)
    cold = run_model(mid_gguf, exact, 130, 100, batches, n_new, 11)
    for a, b in zip(ref[0], cold[0]):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(ref[1], cold[1])
    st, tc = cold[2], cold[3]
    assert st.oversubscribed == 1 and tc.oversubscribed == 1 and ref[2].oversubscribed == 0
    assert st.slots == 130 and st.resident == 130 and st.host_slots == 100 and st.pool == 384
    assert st.fetched > 0 and st.evictions == st.fetched                 # every arrival took a slot from a resident
    assert tc.fetched == st.fetched and tc.fetch_bytes == st.fetched * 512 * 2048 // 32 * 18   # file bytes: 18 per 32
    assert st.lookups == ref[2].lookups                                  # the same reads, wherever they were served
    assert tc.picks_copy_us > 0 and tc.read_us > 0
    assert cold[5]["replays"] == 0 and cold[5]["captures"] == 0          # picks are read back mid-pass: no graph
    assert cold[6] == 0                                                  # migration by counts is paused
    assert "cold" in cold[4] and "the model file" in cold[4]
    # the lookahead read ahead of the layers during decode, and some of its guesses were used
    assert tc.prefetch_reads > 0 and 0 < tc.prefetch_used <= tc.prefetch_reads
    # the same run without the lookahead: same values, nothing read ahead
    plain = run_model(mid_gguf, exact, 130, 100, batches, n_new, 11, prefetch=False)
    assert np.array_equal(ref[1], plain[1]) and plain[3].prefetch_reads == 0
    for a, b in zip(ref[0], plain[0]):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    if exact:
        # with fusion on, a single-token pass is recorded and issued as fused launches at each readback of the picks
        # (still no graph); exact mode's fused and unfused kernels give the same bits
        fused = run_model(mid_gguf, True, 130, 100, batches, n_new, 11, fuse=True)
        assert np.array_equal(ref[1], fused[1])
        assert fused[5]["captures"] == 0 and fused[5]["replays"] == 0 and fused[5]["graph_kernels"] > 0
        assert fused[2].fetched > 0


def test_fast_mode_with_cold_experts_follows_the_oracle(tiny_nvfp4_gguf):
    """Fast mode, fusion on: the single-token passes of an oversubscribed pool are recorded and issued as the decode
    path's fused launches in pieces, one per readback of the picks.  Against the CPU oracle fed the same tokens, pass
    by pass, to the whole-model bound of fast mode (a model is discontinuous at every Q8_0 rounding boundary, so this
    shows that nothing is grossly wrong in any piece, e.g. a piece reading what an earlier piece never wrote)."""
    import inferred_hip as ih
    from oracle import binding as ob
    cfg = ih.tiny_config(seed=1, expert_type=ih.NVFP4)
    one = int(cfg.expert_ff) * int(cfg.n_embd) // 16 * 9
    prompt = prompt_ids(33, 4096, 7)
    om = ob.Model(tiny_nvfp4_gguf); oe = ob.Engine(om, 128)
    be = ih.Hip(exact=False)
    be.set_expert_slots(64); be.set_expert_host_budget(16 * one)        # 192 entries: 64 device, 16 pinned, 112 cold
    hm = ih.Model(tiny_nvfp4_gguf); he = ih.Engine(hm, be, 128)
    rel = lambda a, b: float(np.abs(a - b).max()) / max(1.0, float(np.abs(b).max()))
    lo = oe.forward(prompt); lh = he.forward(prompt)
    assert rel(lh, lo) <= 0.1
    agree, nxt = 0, [int(np.argmax(lo))]
    for step in range(12):
        lo = oe.forward(nxt); lh = he.forward(nxt)
        assert rel(lh, lo) <= 0.1, (step, rel(lh, lo))
        agree += int(np.argmax(lo)) == int(np.argmax(lh))
        nxt = [int(np.argmax(lo))]
    assert agree >= 10, agree
    st, g = be.expert_stats(), be.graph_stats()
    assert st.oversubscribed == 1 and st.fetched > 0 and g["captures"] == 0 and g["graph_kernels"] > 0
    assert be.take_error() is None
    he.close(); hm.close(); be.close(); oe.close(); om.close()


def test_tiny_q8_0_model_with_most_of_the_pool_cold(tiny_gguf):
    """Q8_0 experts (16 experts top-4, 192 entries): 64 device slots, 16 pinned blocks, 112 cold; both modes."""
    import inferred_hip as ih
    cfg = ih.tiny_config(seed=0)
    one = int(cfg.expert_ff) * int(cfg.n_embd) // 32 * 34
    for exact in (False, True):
        ref = run_model(tiny_gguf, exact, None, 0, [10, 40, 2], 12, 5)
        cold = run_model(tiny_gguf, exact, 64, 16, [10, 40, 2], 12, 5, expert_bytes=one)
        for a, b in zip(ref[0], cold[0]):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert np.array_equal(ref[1], cold[1])
        assert cold[2].host_slots == 16 and cold[2].fetched > 0 and cold[2].oversubscribed == 1


def make_tensor(n_in=64, n_out=32, n_expert=12, seed=9):
    from oracle import binding as ob
    orc = ob.Oracle(threads=1)
    wb = q8_0_weights(orc, rng(seed), n_expert * n_out, n_in, std=1.0)
    return orc, wb


def test_gclock_takes_the_idle_slots_and_spares_the_leased_ones():
    """One tensor of 12 experts read out of its mapping (no model file): 4 device slots (experts 0..3), 2 pinned blocks
    (4, 5), 6 cold (6..11).  Every result is checked against the CPU oracle."""
    import inferred_hip as ih
    from oracle import binding as ob
    n_in, n_out, n_expert, n_used = 64, 32, 12, 2
    orc, wb = make_tensor(n_in, n_out, n_expert)
    r = rng(10)
    be = ih.Hip(exact=True)
    be.set_expert_slots(4)
    be.set_expert_host_budget(2 * n_out * n_in // 32 * 34)
    E = ih.experts(wb, ih.Q8_0, n_in, n_out, n_expert)

    def once(ids):
        ids = np.array(ids, np.uint32)
        n_tok = ids.size // n_used
        x = r.standard_normal(n_tok * n_in).astype(np.float32)
        want = np.zeros(ids.size * n_out, np.float32); out = np.zeros_like(want)
        orc.matmul_experts(ob.experts(wb, ih.Q8_0, n_in, n_out, n_expert), ids, n_used, x, want)
        be.begin_pass(n_tok)
        be.matmul_experts(E, ih.Hip.host_route(ids, None, n_used), x, out)
        be.end_pass(); be.host_needs(out)
        assert be.take_error() is None
        assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
        return be.expert_stats()

    st = once([0, 1, 2, 3])                      # device-tier experts only: nothing is fetched, their slots warm up
    assert st.oversubscribed == 1 and st.host_slots == 2 and st.fetched == 0 and st.evictions == 0
    st = once([4, 5])                            # pinned blocks are read in place
    assert st.fetched == 0 and st.hits == 4 and st.lookups == 6
    st = once([8, 9])                            # two cold picks: the hand cools 0..3 once, then takes slots 0 and 1
    assert st.fetched == 2 and st.evictions == 2
    st = once([8, 9, 2, 3])                      # all four in device memory now
    assert st.fetched == 2
    st = once([0, 8])                            # expert 0 lost its slot to 8: it comes back; 8 is leased and stays
    assert st.fetched == 3 and st.evictions == 3
    assert np.array_equal(be.expert_counts(wb, n_expert), np.bincount([0, 1, 2, 3, 4, 5, 8, 9, 8, 9, 2, 3, 0, 8], minlength=n_expert))
    be.close()


def test_a_device_tier_smaller_than_one_decision_is_refused():
    import inferred_hip as ih
    n_in, n_out, n_expert, n_used = 64, 32, 12, 2
    orc, wb = make_tensor(n_in, n_out, n_expert, seed=12)
    be = ih.Hip(exact=True)
    be.set_expert_slots(2)
    be.set_expert_host_budget(1)
    E = ih.experts(wb, ih.Q8_0, n_in, n_out, n_expert)
    ids = np.array([0, 5, 1, 6], np.uint32)      # 0 and 1 hold the two slots and are leased; 5 and 6 are cold
    x = np.zeros(2 * n_in, np.float32); out = np.zeros(4 * n_out, np.float32)
    be.begin_pass(2)
    be.matmul_experts(E, ih.Hip.host_route(ids, None, n_used), x, out)
    be.end_pass()
    err = be.take_error() or ""
    assert "smaller than one layer's picks" in err and "2 device slots" in err
    be.close()


def test_cold_experts_are_read_unbuffered_where_the_file_system_allows(mid_gguf, monkeypatch):
    """The reader threads open the model file a second time with O_DIRECT and read whole 4,096-byte units around an
    expert's bytes into an aligned buffer of their own (/root/reference src/platform.rs:60-96, 200-215;
    src/ops/cuda/fetch.rs:71-73, experts.rs:310-312): on by default, off with INFERRED_FETCH_DIRECT=0, and buffered when
    the file system refuses the flag.  Either way the bytes are the file's: ids and logits bit-identical to the
    all-resident run."""
    batches, n_new = [3, 48], 8
    ref = run_model(mid_gguf, True, None, 0, batches, n_new, 13)
    try:
        fd = os.open(str(mid_gguf), os.O_RDONLY | os.O_DIRECT)
        os.close(fd)
        fs_allows = True
    except OSError:
        fs_allows = False
    for setting in (None, "0", "1"):
        if setting is None:
            monkeypatch.delenv("INFERRED_FETCH_DIRECT", raising=False)
        else:
            monkeypatch.setenv("INFERRED_FETCH_DIRECT", setting)
        cold = run_model(mid_gguf, True, 130, 100, batches, n_new, 13)
        direct, reads = run_model.reads
        print(f"INFERRED_FETCH_DIRECT={setting}: {direct} of {reads} reads unbuffered (file system allows: {fs_allows})", flush=True)
        assert reads > 0 and cold[2].fetched > 0
        assert direct == (reads if (setting != "0" and fs_allows) else 0), (setting, direct, reads)
        for a, b in zip(ref[0], cold[0]):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert np.array_equal(ref[1], cold[1])
