"""TEST INFRASTRUCTURE — ctypes binding of liboracle.so, the CPU oracle.

Only tests, the smoke check and the benchmark's cpu_baseline leg import this.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "liboracle.so"
F32, F16, Q8_0, BF16, NVFP4 = 0, 1, 8, 30, 40
u64, u32, f32, vp = C.c_uint64, C.c_uint32, C.c_float, C.c_void_p


class Weights(C.Structure):
    _fields_ = [("data", vp), ("len", u64), ("ty", u32), ("pooled", u32), ("n_in", u64), ("n_out", u64)]


class Experts(C.Structure):
    _fields_ = [("data", vp), ("len", u64), ("ty", u32), ("_pad", u32), ("n_in", u64), ("n_out", u64),
                ("n_expert", u64), ("scale", vp), ("scale_len", u64)]


class Attn(C.Structure):
    _fields_ = [("q", vp), ("q_len", u64), ("k", vp), ("v", vp), ("kv_len", u64), ("kv_dim", u64), ("n_pos", u64),
                ("head_dim", u64), ("n_head", u64), ("n_head_kv", u64), ("scale", f32)]


class Delta(C.Structure):
    _fields_ = [("q", vp), ("k", vp), ("v", vp), ("alpha", vp), ("beta", vp), ("ssm_a", vp), ("dt_bias", vp),
                ("n_tokens", u64), ("head_k_dim", u64), ("head_v_dim", u64), ("n_k_heads", u64), ("n_v_heads", u64)]


def build() -> None:
    r = subprocess.run(["make", "-C", str(HERE)], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building liboracle.so failed:\n" + r.stdout + r.stderr)


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        build()
    L = C.CDLL(str(LIB_PATH))
    sig = {
        "orc_c_f16_to_f32": (f32, [C.c_uint16]), "orc_c_f32_to_f16": (C.c_uint16, [f32]),
        "orc_c_bf16_to_f32": (f32, [C.c_uint16]), "orc_c_ue4m3_to_f32": (f32, [C.c_uint8]),
        "orc_c_expf": (f32, [f32]), "orc_c_logf": (f32, [f32]),
        "orc_type_bytes": (u64, [u32, u64]), "orc_dequantize": (C.c_int, [u32, vp, u64, vp]),
        "orc_quantize_q8_0": (None, [vp, u64, vp, vp]), "orc_q8_0_blocks": (None, [vp, u64, vp]),
        "orc_dot_q8_0_q8_0": (f32, [vp, u64, vp, vp]), "orc_dot_nvfp4_q8_0": (f32, [vp, u64, vp, vp]),
        "orc_set_threads": (None, [C.c_int]), "orc_get_threads": (C.c_int, []),
        "orc_rms_norm": (None, [vp, u64, vp, u64, f32, vp]),
        "orc_rms_norm_heads": (None, [vp, u64, vp, u64, f32]),
        "orc_matmul": (None, [vp, vp, u64, vp]),
        "orc_matmul_pair": (None, [vp, vp, vp, u64, vp, vp]),
        "orc_rope_neox": (None, [vp, u64, u64, u64, u64, u64, f32]),
        "orc_softmax": (None, [vp, u64, u64]), "orc_attend": (None, [vp, vp]),
        "orc_silu_mul": (None, [vp, vp, u64]), "orc_scale": (None, [vp, u64, f32]),
        "orc_l2_norm_heads": (None, [vp, u64, u64, f32]),
        "orc_ssm_conv": (None, [vp, vp, u64, vp, u64, u64, vp]),
        "orc_gather_chunks": (None, [vp, u64, u64, u64, vp, u64]),
        "orc_scatter_chunks": (None, [vp, u64, u64, u64, u64, vp]),
        "orc_sigmoid_mul": (None, [vp, vp, u64]), "orc_delta_rule": (None, [vp, vp, vp]),
        "orc_add_assign": (None, [vp, vp, u64]), "orc_add_scaled": (None, [vp, vp, u64, f32]),
        "orc_add_scaled_rows": (None, [vp, u64, vp, vp, u64]),
        "orc_add_scaled_sigmoid": (None, [vp, vp, u64, vp]),
        "orc_kv_write": (None, [vp, u64, vp, u64]),
        "orc_route": (None, [vp, u64, u64, u64, vp, vp]),
        "orc_matmul_experts": (None, [vp, vp, u64, u64, vp, u64, vp]),
        "orc_moe_glu": (None, [vp, vp, vp, u64, u64, vp, u64, vp, vp]),
        "orc_moe_finish": (None, [vp, u64, u64, vp, vp, u64, u64, vp, vp, u64]),
        "orc_argmax": (u32, [vp, u64]),
        "orc_model_open": (vp, [C.c_char_p, C.c_char_p, C.c_size_t]), "orc_model_close": (None, [vp]),
        "orc_model_dims": (None, [vp, vp]), "orc_model_decode_weight_bytes": (u64, [vp]),
        "orc_engine_new": (vp, [vp, u64, u64]), "orc_engine_free": (None, [vp]),
        "orc_engine_reset": (None, [vp]), "orc_engine_set_trace": (None, [vp, vp, vp]),
        "orc_engine_pos": (u64, [vp]), "orc_engine_forward": (C.c_int, [vp, vp, u64, vp]),
        "orc_engine_generate": (C.c_int64, [vp, vp, u64, u64, vp, vp]),
        "orc_engine_ssm_state": (vp, [vp, u64, vp]), "orc_engine_conv_state": (vp, [vp, u64, vp]),
        "orc_engine_k_slab": (vp, [vp, u64, vp]), "orc_engine_v_slab": (vp, [vp, u64, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    _lib = L
    return L


def _p(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def weights(data, ty, n_in, n_out) -> Weights:
    return Weights(_p(data), data.nbytes, ty, 0, n_in, n_out)


def experts(data, ty, n_in, n_out, n_expert, scale=None) -> Experts:
    return Experts(_p(data), data.nbytes, ty, 0, n_in, n_out, n_expert, _p(scale) if scale is not None else None,
                   scale.nbytes if scale is not None else 0)


class Oracle:
    """The ops, with the same call shapes as inferred_hip.Hip so tests read alike."""

    def __init__(self, threads: int = 1):
        self.L = lib()
        self.L.orc_set_threads(threads)

    def set_threads(self, n):
        self.L.orc_set_threads(n)

    def rms_norm(self, x, w, eps, out):
        self.L.orc_rms_norm(_p(x), x.size, _p(w), w.size, eps, _p(out))

    def rms_norm_heads(self, x, w, head_dim, eps):
        self.L.orc_rms_norm_heads(_p(x), x.size, _p(w), head_dim, eps)

    def matmul(self, w, x, out):
        self.L.orc_matmul(C.addressof(w), _p(x), x.size, _p(out))

    def matmul_pair(self, a, b, x, oa, ob):
        self.L.orc_matmul_pair(C.addressof(a), C.addressof(b), _p(x), x.size, _p(oa), _p(ob))

    def rope_neox(self, x, pos, head_dim, n_rot, n_heads, theta):
        self.L.orc_rope_neox(_p(x), x.size, pos, head_dim, n_rot, n_heads, theta)

    def softmax(self, x, row):
        self.L.orc_softmax(_p(x), x.size, row)

    def attend(self, q, k, v, kv_dim, n_pos, head_dim, n_head, n_head_kv, scale, out):
        a = Attn(_p(q), q.size, _p(k), _p(v), k.size, kv_dim, n_pos, head_dim, n_head, n_head_kv, scale)
        self.L.orc_attend(C.addressof(a), _p(out))

    def silu_mul(self, gate, up):
        self.L.orc_silu_mul(_p(gate), _p(up), gate.size)

    def sigmoid_mul(self, x, g):
        self.L.orc_sigmoid_mul(_p(x), _p(g), x.size)

    def add_assign(self, a, b):
        self.L.orc_add_assign(_p(a), _p(b), a.size)

    def add_scaled(self, a, b, s):
        self.L.orc_add_scaled(_p(a), _p(b), a.size, s)

    def add_scaled_rows(self, acc, rows, scales):
        self.L.orc_add_scaled_rows(_p(acc), acc.size, _p(rows), _p(scales), scales.size)

    def add_scaled_sigmoid(self, acc, b, logit):
        self.L.orc_add_scaled_sigmoid(_p(acc), _p(b), acc.size, _p(logit))

    def scale(self, buf, s):
        self.L.orc_scale(_p(buf), buf.size, s)

    def l2_norm_heads(self, x, head_dim, eps):
        self.L.orc_l2_norm_heads(_p(x), x.size, head_dim, eps)

    def ssm_conv(self, state, x, weight, kernel, out):
        self.L.orc_ssm_conv(_p(state), _p(x), x.size, _p(weight), weight.size, kernel, _p(out))

    def gather_chunks(self, src, chunk, stride, offset, out):
        self.L.orc_gather_chunks(_p(src), chunk, stride, offset, _p(out), out.size)

    def scatter_chunks(self, src, chunk, stride, offset, dst):
        self.L.orc_scatter_chunks(_p(src), src.size, chunk, stride, offset, _p(dst))

    def delta_rule(self, q, k, v, alpha, beta, ssm_a, dt_bias, dk, dv, n_k, n_v, state, out):
        n_tok = v.size // (n_v * dv)
        d = Delta(_p(q), _p(k), _p(v), _p(alpha), _p(beta), _p(ssm_a), _p(dt_bias), n_tok, dk, dv, n_k, n_v)
        self.L.orc_delta_rule(C.addressof(d), _p(state), _p(out))

    def kv_write(self, slab, offset, src):
        self.L.orc_kv_write(_p(slab), offset, _p(src), src.size)

    def route(self, probs, n_expert, n_used):
        n_tok = probs.size // n_expert
        ids = np.zeros(n_tok * n_used, np.uint32)
        w = np.zeros(n_tok * n_used, np.float32)
        self.L.orc_route(_p(probs), n_tok, n_expert, n_used, _p(ids), _p(w))
        return ids, w

    def matmul_experts(self, w, ids, n_used, x, out):
        self.L.orc_matmul_experts(C.addressof(w), _p(ids), ids.size, n_used, _p(x), x.size, _p(out))

    def moe_glu(self, gate, up, ids, n_used, x, out, scratch):
        self.L.orc_moe_glu(C.addressof(gate), C.addressof(up), _p(ids), ids.size, n_used, _p(x), x.size, _p(out),
                           _p(scratch))

    def moe_finish(self, out, at, n, rows, weights_, n_used, shared, logit, logit_at):
        n_tok = weights_.size // n_used
        self.L.orc_moe_finish(_p(out), at, n, _p(rows), _p(weights_), n_tok, n_used, _p(shared), _p(logit), logit_at)

    def argmax(self, logits) -> int:
        return int(self.L.orc_argmax(_p(logits), logits.size))

    def quantize_q8_0(self, x):
        sc = np.zeros(x.size // 32, np.float32)
        q = np.zeros(x.size, np.int8)
        self.L.orc_quantize_q8_0(_p(x), x.size, _p(sc), _p(q))
        return sc, q

    def q8_0_blocks(self, x):
        out = np.zeros(x.size // 32 * 34, np.uint8)
        self.L.orc_q8_0_blocks(_p(x), x.size, _p(out))
        return out

    def dequantize(self, ty, data, n):
        out = np.zeros(n, np.float32)
        rc = self.L.orc_dequantize(ty, _p(data), n, _p(out))
        if rc:
            raise ValueError(f"unsupported type {ty}")
        return out


class Model:
    def __init__(self, path):
        self.L = lib()
        err = C.create_string_buffer(1024)
        self.h = self.L.orc_model_open(str(path).encode(), err, 1024)
        if not self.h:
            raise RuntimeError(err.value.decode())
        d = (u64 * 10)()
        self.L.orc_model_dims(self.h, d)
        (self.n_layer, self.n_embd, self.n_vocab, self.n_head, self.n_head_kv, self.head_dim, self.n_expert,
         self.n_expert_used, self.expert_ff, self.n_rot) = [int(v) for v in d]

    def decode_weight_bytes(self):
        return int(self.L.orc_model_decode_weight_bytes(self.h))

    def close(self):
        if self.h:
            self.L.orc_model_close(self.h)
            self.h = None


TRACE_FN = C.CFUNCTYPE(None, vp, C.c_char_p, u32, C.POINTER(C.c_float), u64)


class Engine:
    def __init__(self, model: Model, n_ctx: int, max_batch: int = 512):
        self.L = lib()
        self.model = model
        self.h = self.L.orc_engine_new(model.h, n_ctx, max_batch)

    def reset(self):
        self.L.orc_engine_reset(self.h)

    def set_trace(self, fn):
        """fn(name, layer, values) after every named intermediate of a pass; None removes the hook."""
        if fn is None:
            self._trace_cb = None
            self.L.orc_engine_set_trace(self.h, None, None)
            return

        def cb(_user, name, layer, data, n):
            fn(name.decode(), int(layer), np.ctypeslib.as_array(data, shape=(int(n),)).copy())
        self._trace_cb = TRACE_FN(cb)
        self.L.orc_engine_set_trace(self.h, C.cast(self._trace_cb, vp), None)

    @property
    def pos(self):
        return int(self.L.orc_engine_pos(self.h))

    def forward(self, tokens):
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        logits = np.empty(self.model.n_vocab, np.float32)
        rc = self.L.orc_engine_forward(self.h, _p(t), t.size, _p(logits))
        if rc:
            raise RuntimeError(f"oracle forward error {rc}")
        return logits

    def generate(self, prompt, max_new):
        t = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.zeros(max_new, np.uint32)
        logits = np.empty(self.model.n_vocab, np.float32)
        n = self.L.orc_engine_generate(self.h, _p(t), t.size, max_new, _p(out), _p(logits))
        if n < 0:
            raise RuntimeError(f"oracle generate error {n}")
        return out[:n], logits

    def _slab(self, fn, idx, ctype):
        n = u64()
        p = fn(self.h, idx, C.byref(n))
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(ctype)), shape=(n.value,)).copy()

    def ssm_state(self, layer):
        return self._slab(self.L.orc_engine_ssm_state, layer, C.c_float)

    def conv_state(self, layer):
        return self._slab(self.L.orc_engine_conv_state, layer, C.c_float)

    def k_slab(self, slot):
        return self._slab(self.L.orc_engine_k_slab, slot, C.c_uint16)

    def v_slab(self, slot):
        return self._slab(self.L.orc_engine_v_slab, slot, C.c_uint16)

    def close(self):
        if self.h:
            self.L.orc_engine_free(self.h)
            self.h = None
