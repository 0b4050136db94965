"""ctypes binding of libinferred_hip.so — the MI355X backend for the per-token model loop.

The Python layer is plumbing for tests and benchmarks: every op goes straight to the
C ABI declared in include/inferred_hip.h, which mirrors the reference's `trait Ops`
(/root/reference src/ops/mod.rs:489-1426).  There is no CPU fallback: if the shared
library is missing or no gfx950 device is present, construction raises.
"""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

import numpy as np

F32, F16, Q8_0, BF16, NVFP4 = 0, 1, 8, 30, 40
EXACT, NO_GRAPH, NO_FUSE, NO_CHAIN = 1, 2, 4, 8

_HERE = Path(__file__).resolve().parent
# INFERRED_HIP_LIB names another build of the library (comparing two builds on one machine)
LIB_PATH = Path(os.environ.get("INFERRED_HIP_LIB") or _HERE / "libinferred_hip.so")
CSRC = _HERE.parent / "csrc"

c_u64, c_u32, c_f32 = C.c_uint64, C.c_uint32, C.c_float
PF = C.POINTER(C.c_float)


class Weights(C.Structure):
    _fields_ = [("data", C.c_void_p), ("len", c_u64), ("ty", c_u32), ("pooled", c_u32),
                ("n_in", c_u64), ("n_out", c_u64)]


class Experts(C.Structure):
    _fields_ = [("data", C.c_void_p), ("len", c_u64), ("ty", c_u32), ("_pad", c_u32),
                ("n_in", c_u64), ("n_out", c_u64), ("n_expert", c_u64),
                ("scale", C.c_void_p), ("scale_len", c_u64)]


class Attn(C.Structure):
    _fields_ = [("q", C.c_void_p), ("q_len", c_u64), ("k", C.c_void_p), ("v", C.c_void_p),
                ("kv_len", c_u64), ("kv_dim", c_u64), ("n_pos", c_u64), ("head_dim", c_u64),
                ("n_head", c_u64), ("n_head_kv", c_u64), ("scale", c_f32)]


class Delta(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("alpha", C.c_void_p),
                ("beta", C.c_void_p), ("ssm_a", C.c_void_p), ("dt_bias", C.c_void_p),
                ("n_tokens", c_u64), ("head_k_dim", c_u64), ("head_v_dim", c_u64),
                ("n_k_heads", c_u64), ("n_v_heads", c_u64)]


class Route(C.Structure):
    _fields_ = [("kind", c_u32), ("_pad", c_u32), ("ids", C.c_void_p), ("weights", C.c_void_p),
                ("n_used", c_u64), ("n_tok", c_u64)]


class TierCounters(C.Structure):
    _fields_ = [(n, c_u64) for n in ("fetched", "fetch_bytes", "read_us", "upload_us", "writes_us",
                                      "picks_wait_us", "picks_copy_us", "prefetch_reads", "prefetch_used",
                                      "lookups", "host_reads", "slot_bytes", "vram_free", "vram_total",
                                      "mirrors", "mirror_bytes")] + \
               [("oversubscribed", c_u32), ("_pad", c_u32)] + \
               [(n, c_u64) for n in ("slots", "resident_bytes", "weight_bytes", "kv_bytes", "quant_bytes",
                                      "pool_bytes")]


class ExpertStats(C.Structure):
    _fields_ = [(n, c_u64) for n in ("slots", "slot_bytes", "resident", "pool", "host_slots", "evictions",
                                      "fetched", "lookups", "hits")] + [("oversubscribed", c_u32), ("_pad", c_u32)]


class ProfileRow(C.Structure):
    _fields_ = [("name", C.c_char * 48), ("launches", c_u64), ("ms_total", C.c_double), ("bytes_total", c_u64)]


ROUTER_F32 = 0xffffffff   # SynthConfig.router_type: F32 router / shared-gate / ssm alpha, beta matrices


class SynthConfig(C.Structure):
    _fields_ = [(n, c_u64) for n in ("n_layer", "n_embd", "n_vocab", "n_head", "n_head_kv", "head_dim", "n_rot",
                                      "n_expert", "n_expert_used", "expert_ff", "shared_ff", "ssm_d_conv",
                                      "ssm_d_state", "ssm_n_group", "ssm_dt_rank", "full_attention_interval")] + \
               [("rope_theta", c_f32), ("rms_eps", c_f32), ("dense_type", c_u32), ("expert_type", c_u32),
                ("router_type", c_u32), ("shared_type", c_u32), ("seed", c_u64), ("weight_std", c_f32),
                ("n_threads", c_u32)]


# every symbol include/inferred_hip.h declares
EXPORTS = """it_hip_create it_hip_destroy it_hip_take_error it_hip_has_error it_hip_check_expert_types it_hip_rms_norm
it_hip_rms_norm_heads it_hip_matmul it_hip_rope_neox it_hip_softmax it_hip_attend it_hip_silu_mul
it_hip_l2_norm_heads it_hip_ssm_conv it_hip_gather_chunks it_hip_sigmoid_mul it_hip_delta_rule
it_hip_add_assign it_hip_scale it_hip_scatter_chunks it_hip_matmul_pair it_hip_matmul_experts it_hip_moe_glu
it_hip_moe_finish it_hip_route it_hip_add_scaled_rows it_hip_add_scaled_sigmoid it_hip_add_scaled
it_hip_kv_write it_hip_host_wrote it_hip_host_needs it_hip_begin_pass it_hip_end_pass it_hip_forget_state
it_hip_read_state it_hip_read_kv it_hip_device_report it_hip_reserve_activations it_hip_tier_counters
it_hip_config_report it_hip_setup_cost it_hip_prefetch_hint it_hip_set_expert_budget
it_hip_set_expert_host_budget it_hip_set_expert_slots it_hip_set_expert_pool it_hip_expert_stats
it_hip_clock_pick it_hip_argmax it_hip_embed_argmax it_hip_read_tokens it_hip_sync it_hip_profile_begin it_hip_profile_end it_hip_release it_hip_drop_mirrors it_hip_launch_count it_hip_graph_stats it_hip_chain_stats it_hip_fetch_read_counts it_hip_zero_state it_hip_mfma_ceiling it_model_open
it_model_close it_model_dims it_model_decode_weight_bytes it_model_token_macs it_engine_new it_engine_free it_engine_reset
it_engine_set_trace it_engine_pos it_engine_state_sizes it_engine_checkpoint it_engine_restore it_engine_rewind it_engine_forward it_engine_prefill it_engine_generate
it_engine_decode_greedy it_engine_last_error it_engine_ssm_state it_engine_conv_state it_engine_k_slab
it_engine_v_slab it_synth_write_gguf it_hip_attend_noalloc it_hip_reserve_for_weights it_hip_reserve_for_kv
it_hip_set_prefetch it_hip_set_model_path it_hip_set_map_base it_hip_expert_coverage it_hip_replace_experts_by_counts
it_hip_expert_counts it_hip_mean_streams it_hip_mul_rows it_hip_silu it_hip_sigmoid it_hip_mul_streams it_hip_row_dot
it_hip_signed_sqrt_sigmoid it_hip_dilated_conv it_hip_qsa_pool it_hip_qsa_select it_hip_attend_sparse""".split()

_lib = None


def build(verbose: bool = False) -> None:
    """Compile libinferred_hip.so for gfx950 with the Makefile beside the sources."""
    import subprocess
    jobs = min(16, os.cpu_count() or 4)
    r = subprocess.run(["make", "-C", str(CSRC), f"-j{jobs}"], capture_output=True, text=True)
    if verbose or r.returncode != 0:
        print(r.stdout[-4000:], r.stderr[-4000:])
    if r.returncode != 0:
        raise RuntimeError("building libinferred_hip.so failed")


def lib() -> C.CDLL:
    """Load the shared library (never builds it; never falls back to anything else)."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `make -C {CSRC}` (or __graft_entry__.build())")
    L = C.CDLL(str(LIB_PATH))
    vp, u64, u32, f32 = C.c_void_p, c_u64, c_u32, c_f32
    sig = {
        "it_hip_create": (vp, [u32, C.c_int, C.c_char_p, C.c_size_t]),
        "it_hip_has_error": (C.c_int, [vp]),
        "it_hip_embed_argmax": (C.c_int, [vp, vp, vp, u64, vp, u64, u64]),
        "it_hip_read_tokens": (None, [vp, u64, u64, vp]),
        "it_hip_destroy": (None, [vp]),
        "it_hip_take_error": (C.c_int, [vp, C.c_char_p, C.c_size_t]),
        "it_hip_check_expert_types": (C.c_int, [u32, u32, u32, C.c_char_p, C.c_size_t]),
        "it_hip_rms_norm": (None, [vp, vp, u64, vp, u64, f32, vp, u64]),
        "it_hip_rms_norm_heads": (None, [vp, vp, u64, vp, u64, u64, f32]),
        "it_hip_matmul": (None, [vp, vp, vp, u64, vp, u64]),
        "it_hip_rope_neox": (None, [vp, vp, u64, u64, u64, u64, u64, f32]),
        "it_hip_softmax": (None, [vp, vp, u64, u64]),
        "it_hip_attend": (None, [vp, vp, vp, u64]),
        "it_hip_silu_mul": (None, [vp, vp, u64, vp, u64]),
        "it_hip_l2_norm_heads": (None, [vp, vp, u64, u64, f32]),
        "it_hip_ssm_conv": (None, [vp, vp, u64, vp, u64, vp, u64, u64, vp, u64]),
        "it_hip_gather_chunks": (None, [vp, vp, u64, u64, u64, u64, vp, u64]),
        "it_hip_sigmoid_mul": (None, [vp, vp, u64, vp, u64]),
        "it_hip_delta_rule": (None, [vp, vp, vp, u64, vp, u64]),
        "it_hip_add_assign": (None, [vp, vp, u64, vp, u64]),
        "it_hip_scale": (None, [vp, vp, u64, f32]),
        "it_hip_scatter_chunks": (None, [vp, vp, u64, u64, u64, u64, vp, u64]),
        "it_hip_matmul_pair": (None, [vp, vp, vp, vp, u64, vp, u64, vp, u64]),
        "it_hip_matmul_experts": (None, [vp, vp, vp, vp, u64, vp, u64]),
        "it_hip_moe_glu": (None, [vp, vp, vp, vp, vp, u64, vp, u64, vp, u64]),
        "it_hip_moe_finish": (None, [vp, vp, u64, u64, u64, vp, u64, vp, vp, u64, vp, u64, u64]),
        "it_hip_route": (None, [vp, vp, u64, u64, u64, vp]),
        "it_hip_add_scaled_rows": (None, [vp, vp, u64, vp, u64, vp, u64]),
        "it_hip_add_scaled_sigmoid": (None, [vp, vp, u64, vp, u64, vp, u64]),
        "it_hip_add_scaled": (None, [vp, vp, u64, vp, u64, f32]),
        "it_hip_kv_write": (None, [vp, vp, u64, u64, vp, u64]),
        "it_hip_host_wrote": (None, [vp, vp, u64]),
        "it_hip_host_needs": (None, [vp, vp, u64]),
        "it_hip_begin_pass": (None, [vp, u64]),
        "it_hip_end_pass": (None, [vp]),
        "it_hip_forget_state": (None, [vp]),
        "it_hip_read_state": (None, [vp, vp, u64]),
        "it_hip_read_kv": (None, [vp, vp, u64]),
        "it_hip_device_report": (None, [vp]),
        "it_hip_reserve_activations": (None, [vp, u64]),
        "it_hip_tier_counters": (C.c_int, [vp, vp]),
        "it_hip_config_report": (C.c_size_t, [vp, C.c_char_p, C.c_size_t]),
        "it_hip_setup_cost": (u64, [vp, C.c_char_p, C.c_size_t]),
        "it_hip_prefetch_hint": (None, [vp, vp, vp, u64, u64]),
        "it_hip_set_expert_budget": (None, [vp, u64]),
        "it_hip_set_expert_host_budget": (None, [vp, u64]),
        "it_hip_set_expert_slots": (None, [vp, u64]),
        "it_hip_set_expert_pool": (None, [vp, u64]),
        "it_hip_expert_stats": (None, [vp, vp]),
        "it_hip_reserve_for_weights": (None, [vp, u64]),
        "it_hip_reserve_for_kv": (None, [vp, u64]),
        "it_hip_set_prefetch": (None, [vp, C.c_int]),
        "it_hip_set_model_path": (None, [vp, C.c_char_p]),
        "it_hip_set_map_base": (None, [vp, u64]),
        "it_hip_expert_coverage": (C.c_int, [vp, vp, vp]),
        "it_hip_replace_experts_by_counts": (C.c_int64, [vp]),
        "it_hip_expert_counts": (u64, [vp, vp, vp, u64]),
        "it_hip_mean_streams": (None, [vp, vp, u64, u64, u64, f32, vp, u64]),
        "it_hip_mul_rows": (None, [vp, vp, u64, vp, u64]),
        "it_hip_silu": (None, [vp, vp, u64]),
        "it_hip_sigmoid": (None, [vp, vp, u64]),
        "it_hip_mul_streams": (None, [vp, vp, u64, vp, u64, vp, u64, u64]),
        "it_hip_row_dot": (None, [vp, vp, u64, vp, u64, u64, vp, u64]),
        "it_hip_signed_sqrt_sigmoid": (None, [vp, vp, u64]),
        "it_hip_dilated_conv": (None, [vp, vp, u64, vp, u64, vp, u64, u64, u64, vp, u64]),
        "it_hip_qsa_pool": (None, [vp, vp, u64, vp, u64, vp]),
        "it_hip_qsa_select": (None, [vp, vp, u64, vp, u64, vp, vp, u64, vp, u64]),
        "it_hip_attend_sparse": (None, [vp, vp, vp, u64, vp, vp, u64]),
        "it_hip_clock_pick": (C.c_int64, [vp, vp, u64, vp]),
        "it_hip_argmax": (u32, [vp, vp, u64]),
        "it_hip_sync": (None, [vp]),
        "it_hip_profile_begin": (None, [vp]),
        "it_hip_profile_end": (C.c_int, [vp, vp, C.c_int]),
        "it_hip_release": (None, [vp, vp]),
        "it_hip_drop_mirrors": (None, [vp]),
        "it_hip_launch_count": (u64, [vp]),
        "it_hip_graph_stats": (None, [vp, vp]),
        "it_hip_chain_stats": (None, [vp, vp]),
        "it_hip_fetch_read_counts": (None, [vp, vp]),
        "it_model_open": (vp, [C.c_char_p, C.c_char_p, C.c_size_t]),
        "it_hip_mfma_ceiling": (C.c_int, [vp, C.c_int, C.c_int, vp]),
        "it_hip_zero_state": (None, [vp]),
        "it_model_close": (None, [vp]),
        "it_model_dims": (None, [vp, vp]),
        "it_model_decode_weight_bytes": (u64, [vp]),
        "it_model_token_macs": (None, [vp, vp]),
        "it_engine_new": (vp, [vp, vp, u64, u64]),
        "it_engine_free": (None, [vp]),
        "it_engine_reset": (None, [vp]),
        "it_engine_set_trace": (None, [vp, vp, vp]),
        "it_engine_pos": (u64, [vp]),
        "it_engine_state_sizes": (None, [vp, vp]),
        "it_engine_checkpoint": (u64, [vp, vp, vp]),
        "it_engine_restore": (C.c_int, [vp, u64, vp, vp]),
        "it_engine_rewind": (C.c_int, [vp, u64]),
        "it_engine_forward": (C.c_int, [vp, vp, u64, vp]),
        "it_engine_prefill": (C.c_int, [vp, vp, u64, vp]),
        "it_engine_generate": (C.c_int64, [vp, vp, u64, u64, vp, vp]),
        "it_engine_decode_greedy": (C.c_int64, [vp, u64, vp]),
        "it_engine_last_error": (C.c_char_p, [vp]),
        "it_engine_ssm_state": (vp, [vp, u64, vp]),
        "it_engine_conv_state": (vp, [vp, u64, vp]),
        "it_engine_k_slab": (vp, [vp, u64, vp]),
        "it_engine_v_slab": (vp, [vp, u64, vp]),
        "it_synth_write_gguf": (C.c_int, [C.c_char_p, vp, C.c_char_p, C.c_size_t]),
        "it_hip_attend_noalloc": (C.c_int, [vp, vp, u64, vp, C.c_char_p, C.c_size_t]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def _p(a):
    """Address of a contiguous numpy array (the caller keeps it alive)."""
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def weights(data: np.ndarray, ty: int, n_in: int, n_out: int) -> Weights:
    return Weights(_p(data), data.nbytes, ty, 0, n_in, n_out)


def experts(data: np.ndarray, ty: int, n_in: int, n_out: int, n_expert: int, scale: np.ndarray | None = None) -> Experts:
    return Experts(_p(data), data.nbytes, ty, 0, n_in, n_out, n_expert,
                   _p(scale) if scale is not None else None, scale.nbytes if scale is not None else 0)


class HipError(RuntimeError):
    pass


NOALLOC_SCRATCH_BYTES = 8 << 20


def attend_noalloc(q_ptr: int, q_len: int, k_ptr: int, v_ptr: int, kv_len: int, kv_dim: int, n_pos: int,
                   head_dim: int, n_head: int, n_head_kv: int, scale: float, out_ptr: int, out_len: int,
                   stream: int = 0):
    """it_hip_attend_noalloc over DEVICE addresses (q, out: f32; k, v: f16 bits).  Returns (code, message):
    0 = enqueued on `stream`, 1 = bad argument, 2 = too large for the fixed scratch, 3 = device error."""
    a = Attn(q_ptr, q_len, k_ptr, v_ptr, kv_len, kv_dim, n_pos, head_dim, n_head, n_head_kv, scale)
    err = C.create_string_buffer(512)
    rc = lib().it_hip_attend_noalloc(C.addressof(a), out_ptr, out_len, stream, err, 512)
    return int(rc), err.value.decode()


class Hip:
    """One backend instance: `Cuda::new` of the reference, for gfx950."""

    def __init__(self, exact: bool = False, graph: bool = True, device: int = 0, fuse: bool = True, chain: bool = True):
        self.L = lib()
        err = C.create_string_buffer(512)
        flags = (EXACT if exact else 0) | (0 if graph else NO_GRAPH) | (0 if fuse else NO_FUSE) | (0 if chain else NO_CHAIN)
        self.h = self.L.it_hip_create(flags, device, err, 512)
        if not self.h:
            raise HipError(err.value.decode())
        self.exact = exact

    def close(self):
        if self.h:
            self.L.it_hip_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def take_error(self) -> str | None:
        msg = C.create_string_buffer(1024)
        return msg.value.decode() if self.L.it_hip_take_error(self.h, msg, 1024) else None

    def raise_if_error(self):
        e = self.take_error()
        if e:
            raise HipError(e)

    # ---- ops: numpy float32 arrays are the host buffers of the seam ----
    def rms_norm(self, x, w, eps, out):
        self.L.it_hip_rms_norm(self.h, _p(x), x.size, _p(w), w.size, eps, _p(out), out.size)

    def rms_norm_heads(self, x, w, head_dim, eps):
        self.L.it_hip_rms_norm_heads(self.h, _p(x), x.size, _p(w), w.size, head_dim, eps)

    def matmul(self, w: Weights, x, out):
        self.L.it_hip_matmul(self.h, C.addressof(w), _p(x), x.size, _p(out), out.size)

    def matmul_pair(self, a: Weights, b: Weights, x, out_a, out_b):
        self.L.it_hip_matmul_pair(self.h, C.addressof(a), C.addressof(b), _p(x), x.size, _p(out_a), out_a.size,
                                  _p(out_b), out_b.size)

    def rope_neox(self, x, pos, head_dim, n_rot, n_heads, theta):
        self.L.it_hip_rope_neox(self.h, _p(x), x.size, pos, head_dim, n_rot, n_heads, theta)

    def softmax(self, x, row):
        self.L.it_hip_softmax(self.h, _p(x), x.size, row)

    def attend(self, q, k, v, kv_dim, n_pos, head_dim, n_head, n_head_kv, scale, out):
        a = Attn(_p(q), q.size, _p(k), _p(v), k.size, kv_dim, n_pos, head_dim, n_head, n_head_kv, scale)
        self.L.it_hip_attend(self.h, C.addressof(a), _p(out), out.size)

    def silu_mul(self, gate, up):
        self.L.it_hip_silu_mul(self.h, _p(gate), gate.size, _p(up), up.size)

    def sigmoid_mul(self, x, g):
        self.L.it_hip_sigmoid_mul(self.h, _p(x), x.size, _p(g), g.size)

    def add_assign(self, a, b):
        self.L.it_hip_add_assign(self.h, _p(a), a.size, _p(b), b.size)

    def add_scaled(self, a, b, s):
        self.L.it_hip_add_scaled(self.h, _p(a), a.size, _p(b), b.size, s)

    def add_scaled_rows(self, acc, rows, scales):
        self.L.it_hip_add_scaled_rows(self.h, _p(acc), acc.size, _p(rows), rows.size, _p(scales), scales.size)

    def add_scaled_sigmoid(self, acc, b, logit):
        self.L.it_hip_add_scaled_sigmoid(self.h, _p(acc), acc.size, _p(b), b.size, _p(logit), logit.size)

    def scale(self, buf, s):
        self.L.it_hip_scale(self.h, _p(buf), buf.size, s)

    def l2_norm_heads(self, x, head_dim, eps):
        self.L.it_hip_l2_norm_heads(self.h, _p(x), x.size, head_dim, eps)

    def ssm_conv(self, state, x, weight, kernel, out):
        self.L.it_hip_ssm_conv(self.h, _p(state), state.size, _p(x), x.size, _p(weight), weight.size, kernel,
                               _p(out), out.size)

    def gather_chunks(self, src, chunk, stride, offset, out):
        self.L.it_hip_gather_chunks(self.h, _p(src), src.size, chunk, stride, offset, _p(out), out.size)

    def scatter_chunks(self, src, chunk, stride, offset, dst):
        self.L.it_hip_scatter_chunks(self.h, _p(src), src.size, chunk, stride, offset, _p(dst), dst.size)

    def delta_rule(self, q, k, v, alpha, beta, ssm_a, dt_bias, dk, dv, n_k, n_v, state, out):
        n_tok = v.size // (n_v * dv)
        d = Delta(_p(q), _p(k), _p(v), _p(alpha), _p(beta), _p(ssm_a), _p(dt_bias), n_tok, dk, dv, n_k, n_v)
        self.L.it_hip_delta_rule(self.h, C.addressof(d), _p(state), state.size, _p(out), out.size)

    def kv_write(self, slab, offset, src):
        self.L.it_hip_kv_write(self.h, _p(slab), slab.size, offset, _p(src), src.size)

    def route(self, probs, n_expert, n_used) -> Route:
        r = Route()
        self.L.it_hip_route(self.h, _p(probs), probs.size, n_expert, n_used, C.addressof(r))
        return r

    @staticmethod
    def host_route(ids: np.ndarray, weights_: np.ndarray | None, n_used: int) -> Route:
        ids64 = np.ascontiguousarray(ids, dtype=np.uint64)
        r = Route(0, 0, _p(ids64), _p(weights_) if weights_ is not None else None, n_used, ids64.size // n_used)
        r._keep = (ids64, weights_)
        return r

    def matmul_experts(self, w: Experts, route: Route, x, out):
        self.L.it_hip_matmul_experts(self.h, C.addressof(w), C.addressof(route), _p(x), x.size, _p(out), out.size)

    def moe_glu(self, gate: Experts, up: Experts, route: Route, x, out, scratch):
        self.L.it_hip_moe_glu(self.h, C.addressof(gate), C.addressof(up), C.addressof(route), _p(x), x.size,
                              _p(out), out.size, _p(scratch), scratch.size)

    def moe_finish(self, out, at, n, rows, route: Route, shared, logit, logit_at):
        self.L.it_hip_moe_finish(self.h, _p(out), out.size, at, n, _p(rows), rows.size, C.addressof(route),
                                 _p(shared), shared.size, _p(logit), logit.size, logit_at)

    # ---- residency ----
    def host_wrote(self, buf):
        self.L.it_hip_host_wrote(self.h, _p(buf), buf.size)

    def host_needs(self, buf):
        self.L.it_hip_host_needs(self.h, _p(buf), buf.size)

    def begin_pass(self, n):
        self.L.it_hip_begin_pass(self.h, n)

    def end_pass(self):
        self.L.it_hip_end_pass(self.h)

    def forget_state(self):
        self.L.it_hip_forget_state(self.h)

    def zero_state(self):
        self.L.it_hip_zero_state(self.h)

    def read_state(self, host):
        self.L.it_hip_read_state(self.h, _p(host), host.size)

    def read_kv(self, slab):
        self.L.it_hip_read_kv(self.h, _p(slab), slab.size)

    def argmax(self, buf) -> int:
        return int(self.L.it_hip_argmax(self.h, _p(buf), buf.size))

    def sync(self):
        self.L.it_hip_sync(self.h)

    def profile_begin(self):
        self.L.it_hip_profile_begin(self.h)

    def profile_end(self):
        rows = (ProfileRow * 16)()
        n = self.L.it_hip_profile_end(self.h, rows, 16)
        return [dict(name=rows[i].name.decode(), launches=int(rows[i].launches), ms=float(rows[i].ms_total),
                     bytes=int(rows[i].bytes_total)) for i in range(n)]

    def release(self, buf):
        """Forget the device copy of one host buffer (call before the buffer is freed)."""
        self.L.it_hip_release(self.h, _p(buf))

    def drop_mirrors(self):
        self.L.it_hip_drop_mirrors(self.h)

    def launch_count(self) -> int:
        return int(self.L.it_hip_launch_count(self.h))

    def graph_stats(self):
        v = (c_u64 * 4)()
        self.L.it_hip_graph_stats(self.h, v)
        return {"captures": int(v[0]), "replays": int(v[1]), "aborts": int(v[2]), "graph_kernels": int(v[3])}

    def chain_stats(self):
        """Layer chains of the last fused pass: persistent-kernel launches, the layers they cover, enabled, wait bound."""
        v = (c_u64 * 4)()
        self.L.it_hip_chain_stats(self.h, v)
        return {"chains": int(v[0]), "layers": int(v[1]), "enabled": bool(v[2]), "spin_limit": int(v[3])}

    def fetch_read_counts(self):
        """Cold-tier reads from the model file: (through the unbuffered descriptor, in all)."""
        v = (c_u64 * 2)()
        self.L.it_hip_fetch_read_counts(self.h, v)
        return int(v[0]), int(v[1])

    MFMA_KINDS = {"int8_16x16x64": 0, "int8_16x16x32": 1, "f16_32x32x16": 2, "f16_16x16x32": 3, "f32_16x16x4": 4}

    def mfma_ceiling(self, kind: str, iters: int = 20000) -> float:
        """Measured operations per second of back-to-back MFMA instructions of one kind."""
        v = C.c_double(0.0)
        rc = self.L.it_hip_mfma_ceiling(self.h, self.MFMA_KINDS[kind], iters, C.byref(v))
        if rc:
            raise HipError(f"it_hip_mfma_ceiling({kind}) failed with {rc}")
        return float(v.value)

    def tier_counters(self) -> TierCounters:
        t = TierCounters()
        self.L.it_hip_tier_counters(self.h, C.addressof(t))
        return t

    def expert_stats(self) -> ExpertStats:
        s = ExpertStats()
        self.L.it_hip_expert_stats(self.h, C.addressof(s))
        return s

    def set_expert_budget(self, nbytes):
        self.L.it_hip_set_expert_budget(self.h, nbytes)

    def set_expert_host_budget(self, nbytes):
        self.L.it_hip_set_expert_host_budget(self.h, nbytes)

    def set_expert_slots(self, n):
        self.L.it_hip_set_expert_slots(self.h, n)

    def set_expert_pool(self, n):
        self.L.it_hip_set_expert_pool(self.h, n)

    def reserve_for_weights(self, nbytes):
        self.L.it_hip_reserve_for_weights(self.h, nbytes)

    def reserve_for_kv(self, nbytes):
        self.L.it_hip_reserve_for_kv(self.h, nbytes)

    def set_prefetch(self, on):
        self.L.it_hip_set_prefetch(self.h, 1 if on else 0)

    def set_model_path(self, path):
        self.L.it_hip_set_model_path(self.h, str(path).encode())

    def set_map_base(self, base):
        self.L.it_hip_set_map_base(self.h, base)

    def expert_coverage(self):
        """(share of reads taken by the busiest slab-many expert matrices, reads counted), or None before any
        pooled tensor was seen."""
        f, n = C.c_double(0.0), c_u64(0)
        if self.L.it_hip_expert_coverage(self.h, C.byref(f), C.byref(n)):
            return None
        return float(f.value), int(n.value)

    def replace_experts_by_counts(self) -> int:
        return int(self.L.it_hip_replace_experts_by_counts(self.h))

    def expert_counts(self, tensor: np.ndarray, n_expert: int) -> np.ndarray:
        """Per-expert device read counts of one expert tensor (the array its Experts struct points at)."""
        out = np.zeros(n_expert, np.uint32)
        n = self.L.it_hip_expert_counts(self.h, _p(tensor), _p(out), n_expert)
        return out[:int(n)]

    def config_report(self) -> str:
        b = C.create_string_buffer(2048)
        self.L.it_hip_config_report(self.h, b, 2048)
        return b.value.decode()


class Model:
    def __init__(self, path: str):
        self.L = lib()
        err = C.create_string_buffer(1024)
        self.h = self.L.it_model_open(str(path).encode(), err, 1024)
        if not self.h:
            raise HipError(err.value.decode())
        d = (c_u64 * 10)()
        self.L.it_model_dims(self.h, d)
        (self.n_layer, self.n_embd, self.n_vocab, self.n_head, self.n_head_kv, self.head_dim, self.n_expert,
         self.n_expert_used, self.expert_ff, self.n_rot) = [int(v) for v in d]

    def decode_weight_bytes(self) -> int:
        return int(self.L.it_model_decode_weight_bytes(self.h))

    def token_macs(self):
        """(dense, expert gate+up, expert down) multiply-accumulates of one token, output head excluded."""
        v = (c_u64 * 3)()
        self.L.it_model_token_macs(self.h, v)
        return int(v[0]), int(v[1]), int(v[2])

    def close(self):
        if self.h:
            self.L.it_model_close(self.h)
            self.h = None


TRACE_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_char_p, C.c_uint32, C.POINTER(C.c_float), C.c_uint64)


class Engine:
    def __init__(self, model: Model, be: Hip, n_ctx: int, max_batch: int = 512):
        self.L = lib()
        self.model, self.be = model, be
        self.h = self.L.it_engine_new(model.h, be.h, n_ctx, max_batch)
        if not self.h:
            raise HipError("it_engine_new failed")

    def _err(self, rc):
        raise HipError(f"engine error {rc}: {self.L.it_engine_last_error(self.h).decode()}")

    def reset(self):
        self.L.it_engine_reset(self.h)

    def set_trace(self, fn):
        """fn(name, layer, values) after every named intermediate of a pass (Ctx::trace of the reference,
        src/profile.rs:439-456); None removes the hook.  A traced pass reads device buffers mid-pass, so it runs
        eagerly."""
        if fn is None:
            self._trace_cb = None
            self.L.it_engine_set_trace(self.h, None, None)
            return

        def cb(_user, name, layer, data, n):
            fn(name.decode(), int(layer), np.ctypeslib.as_array(data, shape=(int(n),)).copy())
        self._trace_cb = TRACE_FN(cb)
        self.L.it_engine_set_trace(self.h, C.cast(self._trace_cb, C.c_void_p), None)

    @property
    def pos(self) -> int:
        return int(self.L.it_engine_pos(self.h))

    def checkpoint(self):
        """(position, conv slab, ssm slab): Engine::checkpoint of the reference."""
        n = (c_u64 * 2)()
        self.L.it_engine_state_sizes(self.h, n)
        conv, ssm = np.empty(int(n[0]), np.float32), np.empty(int(n[1]), np.float32)
        pos = int(self.L.it_engine_checkpoint(self.h, _p(conv), _p(ssm)))
        return pos, conv, ssm

    def restore(self, ckpt):
        pos, conv, ssm = ckpt
        rc = self.L.it_engine_restore(self.h, pos, _p(conv), _p(ssm))
        if rc:
            self._err(rc)

    def rewind(self, n) -> bool:
        return bool(self.L.it_engine_rewind(self.h, n))

    def forward(self, tokens, want_logits=True):
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        logits = np.empty(self.model.n_vocab, np.float32) if want_logits else None
        rc = self.L.it_engine_forward(self.h, _p(t), t.size, _p(logits))
        if rc:
            self._err(rc)
        return logits

    def prefill(self, tokens, want_logits=True):
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        logits = np.empty(self.model.n_vocab, np.float32) if want_logits else None
        rc = self.L.it_engine_prefill(self.h, _p(t), t.size, _p(logits))
        if rc:
            self._err(rc)
        return logits

    def generate(self, prompt, max_new):
        t = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.zeros(max_new, np.uint32)
        logits = np.empty(self.model.n_vocab, np.float32)
        n = self.L.it_engine_generate(self.h, _p(t), t.size, max_new, _p(out), _p(logits))
        if n < 0:
            self._err(n)
        return out[:n], logits

    def decode_greedy(self, n):
        out = np.zeros(n, np.uint32)
        got = self.L.it_engine_decode_greedy(self.h, n, _p(out))
        if got < 0:
            self._err(got)
        return out[:got]

    def _slab(self, fn, idx, dtype):
        n = c_u64()
        p = fn(self.h, idx, C.byref(n))
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_float if dtype == np.float32 else C.c_uint16)),
                                     shape=(n.value,)).copy()

    def ssm_state(self, layer):
        return self._slab(self.L.it_engine_ssm_state, layer, np.float32)

    def conv_state(self, layer):
        return self._slab(self.L.it_engine_conv_state, layer, np.float32)

    def k_slab(self, slot):
        return self._slab(self.L.it_engine_k_slab, slot, np.uint16)

    def v_slab(self, slot):
        return self._slab(self.L.it_engine_v_slab, slot, np.uint16)

    def close(self):
        if self.h:
            self.L.it_engine_free(self.h)
            self.h = None


# ---- the benchmark configurations as synthetic-model recipes ----
def tiny_config(seed: int = 0, **over) -> SynthConfig:
    """Config 1: 4 layers (3 GDN + 1 attention), hidden 512, vocab 4096, 16 experts top-4, all Q8_0."""
    c = SynthConfig(n_layer=4, n_embd=512, n_vocab=4096, n_head=8, n_head_kv=2, head_dim=64, n_rot=16,
                    n_expert=16, n_expert_used=4, expert_ff=256, shared_ff=256, ssm_d_conv=4, ssm_d_state=64,
                    ssm_n_group=4, ssm_dt_rank=8, full_attention_interval=4, rope_theta=1e6, rms_eps=1e-6,
                    dense_type=Q8_0, expert_type=Q8_0, router_type=Q8_0, seed=seed, weight_std=0.02, n_threads=8)
    for k, v in over.items():
        setattr(c, k, v)
    return c


def big_config(seed: int = 0, n_layer: int = 48, **over) -> SynthConfig:
    """Config 5: the 35B-A3B shape (48 layers 3:1, hidden 2048, 512 experts top-10, NVFP4 experts)."""
    c = SynthConfig(n_layer=n_layer, n_embd=2048, n_vocab=151936, n_head=16, n_head_kv=2, head_dim=256, n_rot=64,
                    n_expert=512, n_expert_used=10, expert_ff=512, shared_ff=512, ssm_d_conv=4, ssm_d_state=128,
                    ssm_n_group=16, ssm_dt_rank=32, full_attention_interval=4, rope_theta=1e7, rms_eps=1e-6,
                    dense_type=Q8_0, expert_type=NVFP4, router_type=Q8_0, seed=seed, weight_std=0.02, n_threads=16)
    for k, v in over.items():
        setattr(c, k, v)
    return c


def synth_write_gguf(path: str, cfg: SynthConfig) -> None:
    err = C.create_string_buffer(512)
    if lib().it_synth_write_gguf(str(path).encode(), C.addressof(cfg), err, 512):
        raise HipError(err.value.decode())
