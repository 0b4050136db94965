"""An independent float64 restatement of the qwen35moe pass, for pinning the ORDER of operations of the model loop.

Nothing here calls the oracle or the HIP library.  The file has two parts:

  * a GGUF v3 writer in plain Python (container facts from /root/reference src/gguf/mod.rs:143-296 and
    src/gguf/metadata.rs:131-205) that stores a hand-sized model with every tensor in F32, so that the only
    difference between this restatement and a loader-driven f32 run is rounding;
  * `F64Model`: the forward pass written from the reference's description of the architecture
    (src/model/qwen35.rs:956-1127 the layer loop, :1138-1223 attention, :1232-1328 the gated delta net,
    :1545-1700 the routed FFN and its shared expert) in numpy float64, token by token, with dense algebra
    (matrix-vector products, explicit softmax) rather than the seam's op sequence.

A loader or loop that applies an op in another order (the gate scale after the silu, rope before the head norm,
softmax over the picks instead of all experts, k/v written after attending, ...) moves the logits by far more
than the f32 rounding this comparison allows.
"""
import struct

import numpy as np

F32 = 0


# --------------------------------------------------------------------------- GGUF writer
def _s(b):
    b = b.encode()
    return struct.pack("<Q", len(b)) + b


def write_gguf(path, arch, kv, tensors, align=32):
    """kv: list of (key, kind, value) with kind in u32 / f32 / str / i32s; tensors: list of (name, ggml dims,
    float32 array in storage order)."""
    out = bytearray()
    out += b"GGUF" + struct.pack("<Iqq", 3, len(tensors), len(kv) + 1)
    out += _s("general.architecture") + struct.pack("<I", 8) + _s(arch)
    for key, kind, v in kv:
        out += _s(f"{arch}.{key}")
        if kind == "u32":
            out += struct.pack("<II", 4, v)
        elif kind == "f32":
            out += struct.pack("<If", 6, v)
        elif kind == "i32s":
            out += struct.pack("<IIQ", 9, 5, len(v)) + struct.pack(f"<{len(v)}i", *v)
        else:
            raise ValueError(kind)
    off = 0
    blobs = []
    for name, dims, a in tensors:
        a = np.ascontiguousarray(a, np.float32)
        assert a.size == int(np.prod(dims)), name
        out += _s(name) + struct.pack("<I", len(dims)) + struct.pack(f"<{len(dims)}q", *dims)
        out += struct.pack("<IQ", F32, off)
        blobs.append((off, a.tobytes()))
        off = (off + a.nbytes + align - 1) // align * align
    out += b"\0" * ((-len(out)) % align)
    data = bytearray(off)
    for o, b in blobs:
        data[o:o + len(b)] = b
    with open(path, "wb") as f:
        f.write(out)
        f.write(data)


# --------------------------------------------------------------------------- the hand-sized model
class Shape:
    n_layer = 2
    interval = 2            # layer 0 recurrent, layer 1 full attention: (il + 1) % interval == 0 (qwen35.rs:329-331)
    n_embd = 32
    n_vocab = 24
    n_head, n_head_kv, head_dim, n_rot = 4, 2, 16, 8
    n_expert, n_used, expert_ff, shared_ff = 4, 2, 16, 24
    d_conv, d_state, dt_rank, n_group = 4, 8, 4, 2   # dk = dv = 8, four value heads over two key heads
    theta, eps = 10000.0, 1e-5

    d_inner = d_state * dt_rank
    key_dim = d_state * n_group
    value_dim = d_inner
    conv_dim = 2 * key_dim + value_dim
    kv_dim = n_head_kv * head_dim


def draw_weights(seed=7):
    """Every tensor of the model as float64-exact float32 values, keyed by GGUF name."""
    S = Shape
    r = np.random.default_rng(seed)

    def mat(n_out, n_in, std=None):
        return (r.standard_normal((n_out, n_in)) * (std or 1.0 / np.sqrt(n_in))).astype(np.float32)

    def vec(n, lo=0.5, hi=1.5):
        return (lo + (hi - lo) * r.random(n)).astype(np.float32)

    W = {"token_embd.weight": mat(S.n_vocab, S.n_embd, 1.0), "output.weight": mat(S.n_vocab, S.n_embd),
         "output.scale": np.array([1.25], np.float32), "output_norm.weight": vec(S.n_embd)}
    for il in range(S.n_layer):
        p = f"blk.{il}."
        W[p + "attn_norm.weight"] = vec(S.n_embd)
        W[p + "post_attention_norm.weight"] = vec(S.n_embd)
        if (il + 1) % S.interval != 0:
            W[p + "attn_qkv.weight"] = mat(S.conv_dim, S.n_embd, 0.5)
            W[p + "attn_gate.weight"] = mat(S.value_dim, S.n_embd, 0.5)
            W[p + "ssm_conv1d.weight"] = mat(S.conv_dim, S.d_conv, 0.6)
            W[p + "ssm_beta.weight"] = mat(S.dt_rank, S.n_embd, 0.4)
            W[p + "ssm_alpha.weight"] = mat(S.dt_rank, S.n_embd, 0.4)
            W[p + "ssm_a"] = (-np.exp(r.standard_normal(S.dt_rank) * 0.5)).astype(np.float32)
            W[p + "ssm_dt.bias"] = (r.standard_normal(S.dt_rank) * 0.5).astype(np.float32)
            W[p + "ssm_norm.weight"] = vec(S.d_state)
            W[p + "ssm_out.weight"] = mat(S.n_embd, S.value_dim)
        else:
            W[p + "attn_q.weight"] = mat(2 * S.head_dim * S.n_head, S.n_embd, 0.4)
            W[p + "attn_k.weight"] = mat(S.kv_dim, S.n_embd, 0.4)
            W[p + "attn_v.weight"] = mat(S.kv_dim, S.n_embd, 0.4)
            W[p + "attn_output.weight"] = mat(S.n_embd, S.head_dim * S.n_head)
            W[p + "attn_q_norm.weight"] = vec(S.head_dim)
            W[p + "attn_k_norm.weight"] = vec(S.head_dim)
        W[p + "ffn_gate_inp.weight"] = mat(S.n_expert, S.n_embd, 0.5)
        W[p + "ffn_gate_exps.weight"] = mat(S.n_expert * S.expert_ff, S.n_embd, 0.4)
        W[p + "ffn_up_exps.weight"] = mat(S.n_expert * S.expert_ff, S.n_embd, 0.4)
        W[p + "ffn_down_exps.weight"] = mat(S.n_expert * S.n_embd, S.expert_ff, 0.4)
        for t in ("gate", "up", "down"):                       # an NVFP4 file's per-expert second scales
            W[p + f"ffn_{t}_exps.scale"] = vec(S.n_expert, 0.4, 2.0)
        W[p + "ffn_gate_shexp.weight"] = mat(S.shared_ff, S.n_embd, 0.4)
        W[p + "ffn_up_shexp.weight"] = mat(S.shared_ff, S.n_embd, 0.4)
        W[p + "ffn_down_shexp.weight"] = mat(S.n_embd, S.shared_ff, 0.4)
        W[p + "ffn_gate_shexp.scale"] = np.array([1.7], np.float32)   # far from 1: the gate scale sits under the silu
        W[p + "ffn_up_shexp.scale"] = np.array([0.6], np.float32)
        W[p + "ffn_down_shexp.scale"] = np.array([1.3], np.float32)
        W[p + "ffn_gate_inp_shexp.weight"] = (r.standard_normal(S.n_embd) * 0.3).astype(np.float32)
    return W


def write_model(path, W):
    S = Shape
    kv = [("block_count", "u32", S.n_layer), ("embedding_length", "u32", S.n_embd),
          ("expert_count", "u32", S.n_expert), ("expert_used_count", "u32", S.n_used),
          ("expert_feed_forward_length", "u32", S.expert_ff),
          ("expert_shared_feed_forward_length", "u32", S.shared_ff),
          ("attention.head_count", "u32", S.n_head), ("attention.head_count_kv", "u32", S.n_head_kv),
          ("attention.key_length", "u32", S.head_dim), ("attention.value_length", "u32", S.head_dim),
          ("attention.layer_norm_rms_epsilon", "f32", S.eps), ("rope.freq_base", "f32", S.theta),
          ("rope.dimension_count", "u32", S.n_rot), ("rope.dimension_sections", "i32s", [2, 1, 1, 0]),
          ("ssm.conv_kernel", "u32", S.d_conv), ("ssm.inner_size", "u32", S.d_inner),
          ("ssm.state_size", "u32", S.d_state), ("ssm.time_step_rank", "u32", S.dt_rank),
          ("ssm.group_count", "u32", S.n_group), ("full_attention_interval", "u32", S.interval)]
    tensors = []
    for name, a in W.items():
        if name.endswith("_exps.weight"):
            n_in = a.shape[1]
            dims = [n_in, a.shape[0] // S.n_expert, S.n_expert]      # ggml order: row length first
        elif a.ndim == 2:
            dims = [a.shape[1], a.shape[0]]
        else:
            dims = [a.shape[0]]
        tensors.append((name, dims, a))
    write_gguf(path, "qwen35moe", kv, tensors)


MISTAKES = ["delta heads grouped by division", "delta read before the update", "rope before the head norm",
            "weights not renormalized over the picks", "shared gate scale after the silu",
            "expert gate scale after the silu", "shared expert not gated by its logit"]


# --------------------------------------------------------------------------- the float64 pass
def _sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def _silu(x):
    return x * _sigmoid(x)


def _f16(x):
    with np.errstate(over="ignore"):
        return np.asarray(x, np.float64).astype(np.float32).astype(np.float16).astype(np.float64)


class F64Model:
    def __init__(self, W, n_ctx, mistake=None):
        """mistake: None, or the name of one deliberate slip (see MISTAKES) used to show that the comparison
        against this model tells the right order from a plausible wrong one."""
        self.mistake = mistake
        self.W = {k: v.astype(np.float64) for k, v in W.items()}
        S = Shape
        self.pos = 0
        self.K = np.zeros((n_ctx, S.kv_dim))
        self.V = np.zeros((n_ctx, S.kv_dim))
        self.conv_state = np.zeros((S.conv_dim, S.d_conv - 1))         # per channel, oldest sample first
        self.ssm = np.zeros((S.dt_rank, S.d_state, S.d_state))          # [value head][value row][key]

    def _rms(self, x, w, eps):
        return x / np.sqrt(np.mean(x * x) + eps) * w

    def _rope(self, heads, pos):
        """NeoX rotation of the first n_rot dims of every head: dim i pairs with i + n_rot / 2."""
        S = Shape
        half = S.n_rot // 2
        out = heads.copy()
        ang = pos * S.theta ** (-2.0 * np.arange(half) / S.n_rot)
        c, s = np.cos(ang), np.sin(ang)
        # the table the f32 path multiplies by is rounded to f32 (src/ops/naive.rs:205-208)
        c, s = c.astype(np.float32).astype(np.float64), s.astype(np.float32).astype(np.float64)
        a, b = heads[:, :half], heads[:, half:2 * half]
        out[:, :half] = a * c - b * s
        out[:, half:2 * half] = a * s + b * c
        return out

    def _gdn(self, p, normed):
        S, W = Shape, self.W
        qkv = W[p + "attn_qkv.weight"] @ normed
        z = W[p + "attn_gate.weight"] @ normed
        alpha = W[p + "ssm_alpha.weight"] @ normed
        beta = W[p + "ssm_beta.weight"] @ normed
        # depthwise causal convolution over [three stored samples, this token], then silu
        window = np.concatenate([self.conv_state, qkv[:, None]], axis=1)
        conv = _silu(np.sum(window * W[p + "ssm_conv1d.weight"], axis=1))
        self.conv_state = window[:, 1:]
        q = conv[:S.key_dim].reshape(S.n_group, S.d_state)
        k = conv[S.key_dim:2 * S.key_dim].reshape(S.n_group, S.d_state)
        v = conv[2 * S.key_dim:].reshape(S.dt_rank, S.d_state)
        q = q / np.maximum(np.linalg.norm(q, axis=1, keepdims=True), S.eps)
        k = k / np.maximum(np.linalg.norm(k, axis=1, keepdims=True), S.eps)
        core = np.zeros((S.dt_rank, S.d_state))
        for h in range(S.dt_rank):
            kh = h % S.n_group                                          # modulo grouping (src/ops/mod.rs:404-413)
            if self.mistake == "delta heads grouped by division":
                kh = h // (S.dt_rank // S.n_group)
            a = alpha[h] + W[p + "ssm_dt.bias"][h]
            g = np.exp(np.log1p(np.exp(a)) * W[p + "ssm_a"][h])
            b = _sigmoid(beta[h])
            St = self.ssm[h] * g                                        # forget first
            delta = b * (v[h] - St @ k[kh])                             # then correct towards v
            St = St + np.outer(delta, k[kh])
            self.ssm[h] = St
            core[h] = St @ (q[kh] / np.sqrt(S.d_state))                 # read with the UPDATED state
            if self.mistake == "delta read before the update":
                core[h] = (self.ssm[h] - np.outer(delta, k[kh])) @ (q[kh] / np.sqrt(S.d_state))
        normed_core = np.stack([self._rms(core[h], W[p + "ssm_norm.weight"], S.eps) for h in range(S.dt_rank)])
        return W[p + "ssm_out.weight"] @ (_silu(z) * normed_core.reshape(-1))

    def _attn(self, p, normed, pos):
        S, W = Shape, self.W
        qg = (W[p + "attn_q.weight"] @ normed).reshape(S.n_head, 2, S.head_dim)   # per head: query, then gate
        q, gate = qg[:, 0], qg[:, 1]
        k = (W[p + "attn_k.weight"] @ normed).reshape(S.n_head_kv, S.head_dim)
        v = (W[p + "attn_v.weight"] @ normed).reshape(S.n_head_kv, S.head_dim)
        q = np.stack([self._rms(h, W[p + "attn_q_norm.weight"], S.eps) for h in q])   # norm before rotation
        k = np.stack([self._rms(h, W[p + "attn_k_norm.weight"], S.eps) for h in k])
        q, k = self._rope(q, pos), self._rope(k, pos)
        if self.mistake == "rope before the head norm":
            q = (W[p + "attn_q.weight"] @ normed).reshape(S.n_head, 2, S.head_dim)[:, 0]
            q = np.stack([self._rms(h, W[p + "attn_q_norm.weight"], S.eps) for h in self._rope(q, pos)])
        self.K[pos] = _f16(k.reshape(-1))                               # the cache is f16
        self.V[pos] = _f16(v.reshape(-1))
        out = np.zeros((S.n_head, S.head_dim))
        group = S.n_head // S.n_head_kv
        for h in range(S.n_head):
            kvh = h // group                                            # division grouping for attention
            Kh = self.K[:pos + 1, kvh * S.head_dim:(kvh + 1) * S.head_dim]
            Vh = self.V[:pos + 1, kvh * S.head_dim:(kvh + 1) * S.head_dim]
            sc = Kh @ q[h] / np.sqrt(S.head_dim)
            w = np.exp(sc - sc.max())
            out[h] = (w / w.sum()) @ Vh
        return W[p + "attn_output.weight"] @ (out * _sigmoid(gate)).reshape(-1)

    def _ffn(self, p, x):
        S, W = Shape, self.W
        logits = W[p + "ffn_gate_inp.weight"] @ x
        probs = np.exp(logits - logits.max())
        probs /= probs.sum()                                            # over ALL experts, before the choice
        picks = np.argsort(-probs, kind="stable")[:S.n_used]
        w = probs[picks] / max(probs[picks].sum(), 6.103515625e-5)
        if self.mistake == "weights not renormalized over the picks":
            w = probs[picks]
        G = W[p + "ffn_gate_exps.weight"].reshape(S.n_expert, S.expert_ff, S.n_embd)
        U = W[p + "ffn_up_exps.weight"].reshape(S.n_expert, S.expert_ff, S.n_embd)
        D = W[p + "ffn_down_exps.weight"].reshape(S.n_expert, S.n_embd, S.expert_ff)
        gs, us, ds = (W[p + f"ffn_{t}_exps.scale"] for t in ("gate", "up", "down"))
        out = np.zeros(S.n_embd)
        for e, we in zip(picks, w):
            h = _silu(G[e] @ x * gs[e]) * (U[e] @ x * us[e])            # second scales on each product's output
            out += we * (D[e] @ h * ds[e])
        sg = W[p + "ffn_gate_shexp.weight"] @ x * W[p + "ffn_gate_shexp.scale"][0]
        su = W[p + "ffn_up_shexp.weight"] @ x * W[p + "ffn_up_shexp.scale"][0]
        sh = W[p + "ffn_down_shexp.weight"] @ (_silu(sg) * su) * W[p + "ffn_down_shexp.scale"][0]
        if self.mistake == "shared gate scale after the silu":
            sg0 = W[p + "ffn_gate_shexp.weight"] @ x
            sh = W[p + "ffn_down_shexp.weight"] @ (_silu(sg0) * W[p + "ffn_gate_shexp.scale"][0] * su) * W[p + "ffn_down_shexp.scale"][0]
        if self.mistake == "expert gate scale after the silu":
            out = np.zeros(S.n_embd)
            for e, we in zip(picks, w):
                out += we * (D[e] @ (_silu(G[e] @ x) * gs[e] * (U[e] @ x * us[e])) * ds[e])
        if self.mistake == "shared expert not gated by its logit":
            return out + sh, picks
        return out + _sigmoid(W[p + "ffn_gate_inp_shexp.weight"] @ x) * sh, picks

    def token(self, tok):
        """One token at the current position; returns (logits, the expert picks of every layer)."""
        S, W = Shape, self.W
        x = W["token_embd.weight"][tok].copy()
        all_picks = []
        for il in range(S.n_layer):
            p = f"blk.{il}."
            normed = self._rms(x, W[p + "attn_norm.weight"], S.eps)
            x = x + (self._gdn(p, normed) if (il + 1) % S.interval != 0 else self._attn(p, normed, self.pos))
            ffn, picks = self._ffn(p, self._rms(x, W[p + "post_attention_norm.weight"], S.eps))
            all_picks.append(picks)
            x = x + ffn
        self.pos += 1
        logits = W["output.weight"] @ self._rms(x, W["output_norm.weight"], S.eps) * W["output.scale"][0]
        return logits, all_picks
