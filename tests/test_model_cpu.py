"""Host logic without a GPU: the synthetic GGUF writer, both loaders, the oracle's model
loop (structural properties the reference asserts on real models, tests/qwen35.rs:93-140,
348-396, tests/kv_cache.rs:45-176), and the C ABI's export table."""
import re
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent


def prompt_ids(n=32, vocab=4096, seed=0):
    return np.random.default_rng(seed).integers(0, vocab, n).astype(np.uint32)


def test_library_exports_every_declared_symbol():
    import inferred_hip as ih
    header = (ROOT / "include" / "inferred_hip.h").read_text()
    declared = set(re.findall(r"\b(it_(?:hip|model|engine|synth)_\w+)\s*\(", header))
    assert declared == set(ih.EXPORTS), declared ^ set(ih.EXPORTS)
    L = ih.lib()
    for name in declared:
        assert hasattr(L, name), name


def test_no_device_means_a_loud_failure_not_a_fallback():
    import torch
    import inferred_hip as ih
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(ih.HipError):
        ih.Hip()


def test_expert_type_check():
    import ctypes as C
    import inferred_hip as ih
    L = ih.lib(); msg = C.create_string_buffer(256)
    assert L.it_hip_check_expert_types(ih.Q8_0, ih.Q8_0, ih.Q8_0, msg, 256) == 0
    assert L.it_hip_check_expert_types(ih.NVFP4, ih.NVFP4, ih.Q8_0, msg, 256) == 0
    assert L.it_hip_check_expert_types(ih.NVFP4, ih.Q8_0, ih.Q8_0, msg, 256) == 1
    assert L.it_hip_check_expert_types(12, 12, 12, msg, 256) == 1 and b"Q8_0 or NVFP4" in msg.value


def test_clock_pick_behaviours():
    # GCLOCK cases of the reference (src/ops/cuda/experts.rs:2260-2409), on the pure function
    import ctypes as C
    import inferred_hip as ih
    L = ih.lib()
    heat = (C.c_uint8 * 4)(0, 2, 1, 0); leased = (C.c_uint8 * 4)(1, 0, 0, 0); hand = C.c_uint64(0)
    assert L.it_hip_clock_pick(heat, leased, 4, C.byref(hand)) == 3          # leased slot 0 skipped, heat drains
    assert list(heat) == [0, 1, 0, 0] and hand.value == 0
    assert L.it_hip_clock_pick(heat, leased, 4, C.byref(hand)) == 2
    full = (C.c_uint8 * 2)(1, 1)
    assert L.it_hip_clock_pick((C.c_uint8 * 2)(0, 0), full, 2, C.byref(hand)) == -1   # a fully leased ring


def test_loaders_agree_on_the_synthetic_file(tiny_gguf, tiny_nvfp4_gguf):
    import inferred_hip as ih
    from oracle import binding as ob
    for p in (tiny_gguf, tiny_nvfp4_gguf):
        a, b = ih.Model(p), ob.Model(p)
        assert (a.n_layer, a.n_embd, a.n_vocab, a.n_head, a.n_head_kv, a.head_dim, a.n_expert, a.n_expert_used,
                a.expert_ff, a.n_rot) == (b.n_layer, b.n_embd, b.n_vocab, b.n_head, b.n_head_kv, b.head_dim,
                                          b.n_expert, b.n_expert_used, b.expert_ff, b.n_rot) == \
               (4, 512, 4096, 8, 2, 64, 16, 4, 256, 16)
        assert a.decode_weight_bytes() == b.decode_weight_bytes()
        a.close(); b.close()


def test_writer_is_deterministic_in_the_seed(tmp_path):
    import inferred_hip as ih
    cfg = ih.tiny_config(seed=5, n_layer=4, n_vocab=256)
    ih.synth_write_gguf(tmp_path / "a.gguf", cfg); ih.synth_write_gguf(tmp_path / "b.gguf", cfg)
    cfg2 = ih.tiny_config(seed=6, n_layer=4, n_vocab=256); ih.synth_write_gguf(tmp_path / "c.gguf", cfg2)
    a, b, c = [(tmp_path / f).read_bytes() for f in ("a.gguf", "b.gguf", "c.gguf")]
    assert a == b and a != c and len(a) == len(c)


def test_loader_refuses_bad_files(tmp_path, tiny_gguf):
    import inferred_hip as ih
    from oracle import binding as ob
    raw = bytearray(tiny_gguf.read_bytes()[:4096])
    bad = tmp_path / "bad.gguf"; bad.write_bytes(b"GGXX" + bytes(raw[4:]))
    for M in (ih.Model, ob.Model):
        with pytest.raises(RuntimeError):
            M(bad)
    trunc = tmp_path / "trunc.gguf"; trunc.write_bytes(tiny_gguf.read_bytes()[:200000])
    for M in (ih.Model, ob.Model):
        with pytest.raises(RuntimeError):
            M(trunc)


def test_oracle_model_structural_properties(tiny_gguf):
    from oracle import binding as ob
    m = ob.Model(tiny_gguf)
    prompt = prompt_ids(40, seed=3)
    e1 = ob.Engine(m, 64); l1 = e1.forward(prompt)
    e2 = ob.Engine(m, 64)
    for t in prompt:
        l2 = e2.forward([t])
    assert np.array_equal(l1, l2)                                   # batched == token by token
    assert np.array_equal(e1.ssm_state(1), e2.ssm_state(1)) and np.array_equal(e1.k_slab(0), e2.k_slab(0))
    e3 = ob.Engine(m, 64, max_batch=16); ids3, _ = e3.generate(prompt, 4)
    e1.reset(); ids1, _ = e1.generate(prompt, 4)
    assert np.array_equal(ids1, ids3)                               # split prefill == single prefill
    ob.lib().orc_set_threads(4)
    e4 = ob.Engine(m, 64); l4 = e4.forward(prompt)
    ob.lib().orc_set_threads(1)
    assert np.array_equal(l1, l4)                                   # threaded == serial
    with pytest.raises(RuntimeError):
        ob.Engine(m, 8).forward(prompt_ids(9))                      # context overflow
    assert np.isfinite(l1).all() and np.abs(l1).max() > 0.1


def test_oracle_greedy_run_is_reproducible(tiny_gguf):
    from oracle import binding as ob
    m = ob.Model(tiny_gguf)
    a, _ = ob.Engine(m, 128).generate(prompt_ids(), 64)
    b, _ = ob.Engine(m, 128).generate(prompt_ids(), 64)
    assert len(a) == 64 and np.array_equal(a, b) and len(set(a.tolist())) > 8


def _gguf_with_one_tensor(path, dims, ty, offset, extra_kv=b"", n_kv=1, pad_data=4096):
    """A minimal GGUF v3 file: the architecture key (plus raw extra key/value bytes) and one tensor entry whose
    dims, type and offset the caller chooses, followed by pad_data bytes of data."""
    import struct

    def s(b):
        return struct.pack("<Q", len(b)) + b
    out = bytearray(b"GGUF" + struct.pack("<Iqq", 3, 1, n_kv))
    out += s(b"general.architecture") + struct.pack("<I", 8) + s(b"qwen35moe") + extra_kv
    out += s(b"token_embd.weight") + struct.pack("<I", len(dims)) + struct.pack(f"<{len(dims)}q", *dims)
    out += struct.pack("<IQ", ty, offset & (2 ** 64 - 1))
    out += b"\0" * ((-len(out)) % 32) + b"\0" * pad_data
    path.write_bytes(bytes(out))
    return path


def test_reader_checks_file_supplied_sizes_without_wrapping(tmp_path):
    """Sizes read from the file (dims, offsets, array lengths) are combined with checked arithmetic: a product or
    sum that wraps round 64 bits must not pass the bounds test (a tensor pointer outside the mapping would follow)."""
    import struct
    import inferred_hip as ih
    cases = {
        # 2^33 x 2^33 F32 elements: the product wraps to 0 elements
        "dims": (_gguf_with_one_tensor(tmp_path / "dims.gguf", [1 << 33, 1 << 33], 0, 0), "overflows"),
        # 2^62 F32 elements: the byte count wraps
        "bytes": (_gguf_with_one_tensor(tmp_path / "bytes.gguf", [1 << 62], 0, 0), "overflows"),
        # an offset just below 2^64: data_start + offset + size wraps to a small number
        "offset": (_gguf_with_one_tensor(tmp_path / "offset.gguf", [64], 0, -64), "past the end"),
        # an honest tensor that simply does not fit
        "long": (_gguf_with_one_tensor(tmp_path / "long.gguf", [1 << 20], 0, 0), "past the end"),
        # a u8 array whose length times its width wraps / exceeds the file
        "array": (_gguf_with_one_tensor(tmp_path / "array.gguf", [64], 0, 0, n_kv=2,
                                        extra_kv=struct.pack("<Q", 1) + b"k" + struct.pack("<IIQ", 9, 10, 1 << 62)),
                  "overflows"),
        "i32 array": (_gguf_with_one_tensor(tmp_path / "i32.gguf", [64], 0, 0, n_kv=2,
                                            extra_kv=struct.pack("<Q", 1) + b"k" + struct.pack("<IIQ", 9, 5, 1 << 61)),
                      "longer than the file"),
    }
    for name, (path, want) in cases.items():
        with pytest.raises(RuntimeError) as e:
            ih.Model(path)
        assert want in str(e.value), (name, str(e.value))
    from oracle import binding as ob
    for name in ("dims", "bytes", "offset", "long"):
        with pytest.raises(RuntimeError):
            ob.Model(cases[name][0])
