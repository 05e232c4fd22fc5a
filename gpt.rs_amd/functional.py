"""PTIR emitters for the LM path, op for op as the reference's functionals emit them.

Each function appends to the FunctionBuilder that owns its operands, in the evaluation
order of the cited Rust closure, so the instruction stream handed to `run_program` has
the same shape the reference front end produces (before its optimizer).  Reference:
crates/gpt-rs/src/ops/functional/{linalg,normalization,activation,embedding,tensor_ops,
rotary,attention,common}.rs.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import numpy as np

from .ptir import Tensor, TensorSpec


# --------------------------------------------------------------------------- basics
def matmul(a: Tensor, b: Tensor, out_dtype: Optional[str] = None) -> Tensor:
    """ops/functional/linalg.rs:109-127; `out_dtype` sets DotGeneralSpec.out_dtype (spec.rs:354-361)."""
    return a.matmul(b, out_dtype)


def add_bias(x: Tensor, bias: Tensor) -> Tensor:
    """ops/functional/tensor_ops.rs:42-56: x + broadcast(bias)."""
    return x + bias.broadcast_to(x.dims)


def linear(x: Tensor, weight: Tensor, bias: Optional[Tensor] = None, out_dtype: Optional[str] = None) -> Tensor:
    """nn/layers/linear.rs:50-71: x[T,in] . W[in,out] (+ b).  `out_dtype`: the product leaves the f32 accumulator in that
    dtype (docs/backend.md:104-115) instead of x's."""
    if x.spec.rank != 2:
        raise ValueError(f"linear expects 2D input, got shape {x.dims}")
    if x.dims[1] != weight.dims[0]:
        raise ValueError(f"input features ({x.dims[1]}) must match weight rows ({weight.dims[0]})")
    out = matmul(x, weight, out_dtype)
    if bias is not None:
        out = add_bias(out, bias)
    return out


# --------------------------------------------------------------------------- weight-only quantisation
# Build-defined extension (the reference has no quantisation scheme: docs/backend.md:620-632 leaves
# Quantize/Dequantize backend-defined and ref-cpu answers Unimplemented).  Two symmetric schemes:
#   "w8":     int8, one scale per output column:  s_n = bf16(max_k |W[k,n]| / 127), q = clamp(rint(W / s_n), +-127)
#   "w4g128": int4, groups of 128 along K:        s[g,n] = bf16(max |w| / 7), q in [-7, 7], two codes per byte
#             along K: byte[k/2, n] = (q[k] & 0xF) | ((q[k+1] & 0xF) << 4)
# Scales carry the float dtype of the weights they came from.
QUANT_SCHEMES = ("w8", "w4g128")


def _scheme(scheme: str) -> str:
    if scheme not in QUANT_SCHEMES:
        raise ValueError(f"unknown quantisation scheme {scheme!r}; expected one of {QUANT_SCHEMES}")
    return scheme


def quantize_weight(w: Tensor, scheme: str) -> Tuple[Tensor, Tensor]:
    """(codes, scales) of W[K,N] in `scheme`, computed on the device."""
    _scheme(scheme)
    if w.spec.rank != 2:
        raise ValueError(f"quantize_weight expects a matrix, got shape {w.dims}")
    K, N = w.dims
    if scheme == "w8":
        s = w.fb.custom_call("gpt_rs.hip.quantize_w8_scales.v1", [w], TensorSpec(w.dtype, [N]))
        q = w.fb.custom_call("gpt_rs.hip.quantize_w8.v1", [w, s], TensorSpec("Si8", [K, N]))
    else:
        if K % 128:
            raise ValueError(f"w4g128 needs K to be a multiple of 128, got {K}")
        s = w.fb.custom_call("gpt_rs.hip.quantize_w4g128_scales.v1", [w], TensorSpec(w.dtype, [K // 128, N]))
        q = w.fb.custom_call("gpt_rs.hip.quantize_w4g128.v1", [w, s], TensorSpec("Ui8", [K // 2, N]))
    return q, s


def dequantize_weight(q: Tensor, s: Tensor) -> Tensor:
    """W[K,N] = codes * scales in the scales' dtype; the scheme follows from the code dtype."""
    if q.dtype == "Si8":
        return q.fb.custom_call("gpt_rs.hip.dequantize_w8.v1", [q, s], TensorSpec(s.dtype, q.dims))
    if q.dtype == "Ui8":
        return q.fb.custom_call("gpt_rs.hip.dequantize_w4g128.v1", [q, s], TensorSpec(s.dtype, [q.dims[0] * 2, q.dims[1]]))
    raise ValueError(f"codes must be Si8 (w8) or Ui8 (w4g128), got {q.dtype}")


def linear_quantized(x: Tensor, q: Tensor, s: Tensor, bias: Optional[Tensor] = None, out_dtype: Optional[str] = None) -> Tensor:
    """x[T,K] . dequantise(q, s)[K,N] (+ b) without materialising the matrix: f32 accumulation, result in x's dtype
    (or in `out_dtype`, the declared dtype of the call's output)."""
    if x.spec.rank != 2:
        raise ValueError(f"linear expects 2D input, got shape {x.dims}")
    if q.dtype == "Si8":
        target, k = "gpt_rs.hip.dot_w8.v1", q.dims[0]
    elif q.dtype == "Ui8":
        target, k = "gpt_rs.hip.dot_w4g128.v1", q.dims[0] * 2
    else:
        raise ValueError(f"codes must be Si8 (w8) or Ui8 (w4g128), got {q.dtype}")
    if x.dims[1] != k:
        raise ValueError(f"input features ({x.dims[1]}) must match weight rows ({k})")
    out = x.fb.custom_call(target, [x, q, s], TensorSpec(out_dtype or x.dtype, [x.dims[0], q.dims[1]]))
    if bias is not None:
        out = add_bias(out, bias)
    return out


def embedding_lookup(weight: Tensor, indices: Tensor) -> Tensor:
    """ops/functional/embedding.rs:37-54."""
    if indices.spec.rank != 1:
        raise ValueError("embedding indices must be rank 1")
    return weight.take(indices)


# --------------------------------------------------------------------------- norms
def layer_norm(x: Tensor, gamma: Tensor, beta: Tensor, eps: float) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """ops/functional/normalization.rs:123-174.  Returns (out, normalized, mean, inv_std)."""
    fb = x.fb
    axis = x.spec.rank - 1
    n = x.dims[axis]
    red = tuple(x.dims[:-1]) + (1,)
    s = x.reduce_sum([axis], True)
    inv_count = fb.scalar_broadcast(float(np.float32(1.0) / np.float32(n)), red, x.dtype)
    mean = s * inv_count
    mean_b = mean.broadcast_to(x.dims)
    centered = x - mean_b
    centered_sq = centered * centered
    var_sum = centered_sq.reduce_sum([axis], True)
    var_mean = var_sum * inv_count
    var_eps = var_mean + fb.scalar_broadcast(eps, red, x.dtype)
    inv_std = var_eps.rsqrt()
    inv_std_b = inv_std.broadcast_to(x.dims)
    normalized = centered * inv_std_b
    gamma_b = gamma.broadcast_to(x.dims)
    beta_b = beta.broadcast_to(x.dims)
    out = normalized * gamma_b + beta_b
    return out, normalized, mean, inv_std


def rms_norm(x: Tensor, gamma: Tensor, eps: float) -> Tuple[Tensor, Tensor, Tensor]:
    """ops/functional/normalization.rs:183-217.  Returns (out, normalized, inv_rms)."""
    fb = x.fb
    axis = x.spec.rank - 1
    n = x.dims[axis]
    red = tuple(x.dims[:-1]) + (1,)
    squared = x * x
    s = squared.reduce_sum([axis], True)
    inv_count = fb.scalar_broadcast(float(np.float32(1.0) / np.float32(n)), red, x.dtype)
    mean_square = s * inv_count
    inv_rms = (mean_square + fb.scalar_broadcast(eps, red, x.dtype)).rsqrt()
    normalized = x * inv_rms.broadcast_to(x.dims)
    gamma_b = gamma.broadcast_to(x.dims)
    out = normalized * gamma_b
    return out, normalized, inv_rms


# --------------------------------------------------------------------------- activations
def softmax_last_axis(x: Tensor, axis: Optional[int] = None) -> Tensor:
    """ops/functional/common.rs:22-31 (division by the broadcast sum, not reciprocal-multiply)."""
    axis = x.spec.rank - 1 if axis is None else axis
    m = x.reduce_max([axis], True)
    shifted = x - m.broadcast_to(x.dims)
    e = shifted.exp()
    s = e.reduce_sum([axis], True)
    return e / s.broadcast_to(x.dims)


def gelu(x: Tensor) -> Tensor:
    """ops/functional/activation.rs:96-113: exact-erf GELU; sqrt(2) folded on the host as f32."""
    half = 0.5 * x
    scaled = x / float(np.sqrt(np.float32(2.0)))
    erf = scaled.erf()
    one_plus = 1.0 + erf
    return half * one_plus


def silu(x: Tensor) -> Tensor:
    """ops/functional/activation.rs:119-134."""
    neg = x * -1.0
    e = neg.exp()
    denom = 1.0 + e
    return x / denom


def swiglu(gate: Tensor, up: Tensor) -> Tensor:
    """ops/functional/activation.rs:141-162: silu(gate) * up."""
    if gate.spec != up.spec:
        raise ValueError("swiglu gate/up spec mismatch")
    return silu(gate) * up


# --------------------------------------------------------------------------- RoPE
@dataclass
class YarnScaling:
    """RopeScaling::Yarn (ops/functional/rotary.rs:29-43); unset fields take the reference's defaults."""

    factor: float
    original_max_position_embeddings: int
    mscale: Optional[float] = None
    mscale_all_dim: Optional[float] = None
    beta_fast: Optional[float] = None
    beta_slow: Optional[float] = None
    truncate: bool = True


@dataclass
class RopeConfig:
    """ops/functional/rotary.rs:49-67 (scaling: None | ("linear", factor) | YarnScaling)."""

    rotary_dim: int = 128
    theta: float = 10_000.0
    scaling: Optional[object] = None


def _yarn_inv_freqs(cfg: RopeConfig, y: YarnScaling) -> Tuple[np.ndarray, np.float32]:
    """ops/functional/rotary.rs:102-190, every step in f32: blend of the extrapolated (base) and interpolated
    (base / factor) inverse frequencies over a linear ramp between the correction dims of beta_fast and
    beta_slow, and the attention magnitude 0.1 * mscale * ln(factor) + 1."""
    f32 = np.float32
    factor = f32(y.factor)
    if not (np.isfinite(factor) and factor > 0):
        raise ValueError(f"rope yarn factor must be finite and positive (got {y.factor})")
    if y.original_max_position_embeddings is None or y.original_max_position_embeddings <= 0:
        raise ValueError("rope yarn original_max_position_embeddings must be > 0")
    beta_fast = f32(32.0 if y.beta_fast is None else y.beta_fast)
    beta_slow = f32(1.0 if y.beta_slow is None else y.beta_slow)
    if not (np.isfinite(beta_fast) and np.isfinite(beta_slow) and beta_fast >= beta_slow):
        raise ValueError(f"rope yarn beta range is invalid: beta_fast={beta_fast} beta_slow={beta_slow}")

    def get_mscale(scale, mscale):
        return f32(1.0) if scale <= 1.0 else f32(f32(f32(0.1) * f32(mscale)) * np.log(scale, dtype=np.float32)) + f32(1.0)

    if y.mscale is not None and y.mscale_all_dim is not None and y.mscale != 0.0 and y.mscale_all_dim != 0.0:
        magnitude = f32(get_mscale(factor, y.mscale) / get_mscale(factor, y.mscale_all_dim))
    else:
        magnitude = f32(get_mscale(factor, 1.0))
    if not (np.isfinite(magnitude) and magnitude > 0):
        raise ValueError(f"rope yarn magnitude must be finite and positive (got {magnitude})")
    rot, theta = f32(cfg.rotary_dim), f32(cfg.theta)
    orig = f32(y.original_max_position_embeddings)

    def correction_dim(num_rotations):
        return f32(f32(rot * np.log(f32(orig / f32(f32(num_rotations * f32(2.0)) * f32(np.pi))), dtype=np.float32))
                   / f32(f32(2.0) * np.log(theta, dtype=np.float32)))

    low, high = correction_dim(beta_fast), correction_dim(beta_slow)
    if y.truncate:
        low, high = f32(np.floor(low)), f32(np.ceil(high))
    low = f32(max(low, f32(0.0)))
    high = f32(min(high, f32(max(cfg.rotary_dim - 1, 0))))
    ramp_max = high
    if abs(f32(low - ramp_max)) < np.finfo(np.float32).eps:
        ramp_max = f32(ramp_max + f32(0.001))
    i = np.arange(cfg.rotary_dim // 2, dtype=np.float32)
    base = np.power(theta, (f32(2.0) * i) / rot, dtype=np.float32)
    extrapolation = (f32(1.0) / base).astype(np.float32)
    interpolation = (f32(1.0) / (factor * base).astype(np.float32)).astype(np.float32)
    ramp = np.clip(((i - low) / f32(ramp_max - low)).astype(np.float32), f32(0.0), f32(1.0))
    extrapolation_factor = (f32(1.0) - ramp).astype(np.float32)
    inv = (interpolation * (f32(1.0) - extrapolation_factor) + extrapolation * extrapolation_factor).astype(np.float32)
    return inv, magnitude


def rotary_cos_sin_cache_slice(start: int, length: int, cfg: RopeConfig) -> Tuple[np.ndarray, np.ndarray]:
    """Host-side f32 tables [len, rotary_dim/2] (ops/functional/rotary.rs:75-230).

    inv_freq_i = theta^(-(2i)/rot) via f32 powf, angle = (pos as f32) * inv_freq,
    all arithmetic in f32 as the reference does.
    """
    if cfg.rotary_dim <= 0 or cfg.rotary_dim % 2:
        raise ValueError(f"rotary_dim must be a positive even number (got {cfg.rotary_dim})")
    if not (math.isfinite(cfg.theta) and cfg.theta > 0):
        raise ValueError(f"theta must be finite and positive (got {cfg.theta})")
    half = cfg.rotary_dim // 2
    i = np.arange(half, dtype=np.float32)
    exponent = (np.float32(2.0) * i) / np.float32(cfg.rotary_dim)
    inv = np.power(np.float32(cfg.theta), -exponent, dtype=np.float32)
    magnitude = np.float32(1.0)
    if isinstance(cfg.scaling, YarnScaling):
        inv, magnitude = _yarn_inv_freqs(cfg, cfg.scaling)
    elif cfg.scaling is not None:
        kind, factor = cfg.scaling
        if kind != "linear":
            raise NotImplementedError(f"rope scaling {kind}")
        if not (math.isfinite(factor) and factor > 0):
            raise ValueError(f"rope scaling factor must be finite and positive (got {factor})")
        inv = (inv / np.float32(factor)).astype(np.float32)
    pos = np.arange(start, start + length, dtype=np.float32)[:, None]
    angle = (pos * inv[None, :]).astype(np.float32)
    return (np.cos(angle).astype(np.float32) * magnitude).astype(np.float32), (np.sin(angle).astype(np.float32) * magnitude).astype(np.float32)


@dataclass
class AttentionConfig:
    """ops/functional/attention.rs AttentionConfig."""

    embed_dim: int
    num_query_heads: int
    num_key_value_heads: int
    head_dim: int
    kv_head_dim: Optional[int] = None

    def __post_init__(self):
        if self.kv_head_dim is None:
            self.kv_head_dim = self.head_dim
        if self.num_query_heads % self.num_key_value_heads:
            raise ValueError("num_query_heads must be a multiple of num_key_value_heads")

    @property
    def kv_group_size(self): return self.num_query_heads // self.num_key_value_heads
    @property
    def query_projection_dim(self): return self.num_query_heads * self.head_dim
    @property
    def key_value_projection_dim(self): return self.num_key_value_heads * self.kv_head_dim
    @property
    def total_projection_dim(self): return self.query_projection_dim + 2 * self.key_value_projection_dim


def _rope_heads(x_slice: Tensor, cos: Tensor, sin: Tensor, seq: int, heads: int, head_dim: int,
                half: int) -> Tensor:
    rot = 2 * half
    cos_h = cos.reshape([1, seq, half]).broadcast_to([heads, seq, half])
    sin_h = sin.reshape([1, seq, half]).broadcast_to([heads, seq, half])
    xh = x_slice.reshape([seq, heads, head_dim]).transpose([1, 0, 2])
    x_rot = xh.slice([0, 0, 0], [heads, seq, rot])
    first = x_rot.slice([0, 0, 0], [heads, seq, half])
    second = x_rot.slice([0, 0, half], [heads, seq, half])
    first_rot = first * cos_h - second * sin_h
    second_rot = second * cos_h + first * sin_h
    x_rot = Tensor.concat(2, [first_rot, second_rot])
    if rot != head_dim:
        x_pass = xh.slice([0, 0, rot], [heads, seq, head_dim - rot])
        x_rot = Tensor.concat(2, [x_rot, x_pass])
    return x_rot.transpose([1, 0, 2]).reshape([seq, heads * head_dim])


def apply_rope_qkv_packed(cfg: AttentionConfig, qkv: Tensor, cos: Tensor, sin: Tensor) -> Tensor:
    """ops/functional/rotary.rs:430-536: rotate-half RoPE on packed [T, Q|K|V]; V untouched."""
    seq = qkv.dims[0]
    if cos.dims != sin.dims or cos.dims[0] != seq:
        raise ValueError("rope cos/sin shape must be [seq, rotary/2]")
    half = cos.dims[1]
    rot = 2 * half
    if not (0 < rot <= cfg.head_dim) or rot > cfg.kv_head_dim:
        raise ValueError("rope rotary dimension out of range")
    qp, kp = cfg.query_projection_dim, cfg.key_value_projection_dim
    q_slice = qkv.slice([0, 0], [seq, qp])
    k_slice = qkv.slice([0, qp], [seq, kp])
    v_slice = qkv.slice([0, qp + kp], [seq, kp])
    q_flat = _rope_heads(q_slice, cos, sin, seq, cfg.num_query_heads, cfg.head_dim, half)
    k_flat = _rope_heads(k_slice, cos, sin, seq, cfg.num_key_value_heads, cfg.kv_head_dim, half)
    return Tensor.concat(1, [q_flat, k_flat, v_slice])


# --------------------------------------------------------------------------- attention
def _group_kv(t: Tensor, hkv: int, group: int, hq: int, length: int, dh: int) -> Tensor:
    return (t.reshape([hkv, 1, length, dh]).broadcast_to([hkv, group, length, dh])
             .reshape([hq, length, dh]))


def attention(cfg: AttentionConfig, qkv: Tensor,
              cache: Optional[Tuple[Tensor, Tensor]] = None) -> Tuple[Tensor, Tensor, Tensor]:
    """ops/functional/attention.rs:338-541: prefill / concat-cache causal attention.

    Returns (context [T, q_proj], keys [Hkv, Ttot, Dh], values [Hkv, Ttot, Dh]).
    """
    fb = qkv.fb
    seq = qkv.dims[0]
    cache_len = cache[0].dims[1] if cache is not None else 0
    total = cache_len + seq
    hq, hkv, dh, kdh = cfg.num_query_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.kv_head_dim
    group, qp, kp = cfg.kv_group_size, cfg.query_projection_dim, cfg.key_value_projection_dim
    if qkv.dims[1] != cfg.total_projection_dim:
        raise ValueError("qkv last dim must equal total projection dim")

    q_slice = qkv.slice([0, 0], [seq, qp])
    k_slice = qkv.slice([0, qp], [seq, kp])
    v_slice = qkv.slice([0, qp + kp], [seq, kp])
    q_heads = q_slice.reshape([seq, hq, dh]).transpose([1, 0, 2])
    new_k = k_slice.reshape([seq, hkv, kdh]).transpose([1, 0, 2])
    new_v = v_slice.reshape([seq, hkv, kdh]).transpose([1, 0, 2])
    if cache is not None:
        k_all = Tensor.concat(1, [cache[0], new_k])
        v_all = Tensor.concat(1, [cache[1], new_v])
    else:
        k_all, v_all = new_k, new_v
    k_grouped = _group_kv(k_all, hkv, group, hq, total, kdh)
    v_grouped = _group_kv(v_all, hkv, group, hq, total, kdh)
    scores = q_heads.dot_general(k_grouped, [0], [2], [2])
    scale = fb.scalar_broadcast(float(np.float32(1.0) / np.sqrt(np.float32(dh))), [hq, seq, total], qkv.dtype)
    scaled = scores * scale
    positions = fb.iota([total, total], 1)
    query_pos = fb.iota([total, total], 0)
    allowed = query_pos.greater_equal(positions)
    zero = fb.scalar_broadcast(0.0, [total, total], qkv.dtype)
    neg_large = fb.scalar_broadcast(-1e9, [total, total], qkv.dtype)
    base_mask = Tensor.select(allowed, zero, neg_large)
    sliced_mask = base_mask.slice([cache_len, 0], [seq, total])
    mask = sliced_mask.broadcast_to([hq, seq, total])
    masked = scaled + mask
    probs = softmax_last_axis(masked, 2)
    context = probs.dot_general(v_grouped, [0], [2], [1])
    context_out = context.transpose([1, 0, 2]).reshape([seq, qp])
    return context_out, k_all, v_all


def attention_decode_cache(cfg: AttentionConfig, qkv: Tensor, cache_keys: Tensor, cache_values: Tensor,
                           update_starts: Tensor, query_start: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """ops/functional/attention.rs:657-779: T=1 decode over a fixed-capacity KV cache.

    update_starts = si32[3] [0, pos, 0]; query_start = si32[1] [pos].
    Returns (context [1, q_proj], keys', values') -- the caches are program results.
    """
    fb = qkv.fb
    seq = qkv.dims[0]
    if seq != 1:
        raise ValueError("attention_decode_cache supports seq_len == 1 only")
    hq, hkv, dh, kdh = cfg.num_query_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.kv_head_dim
    group, qp, kp = cfg.kv_group_size, cfg.query_projection_dim, cfg.key_value_projection_dim
    cap = cache_keys.dims[1]
    if cache_keys.dims != (hkv, cap, kdh) or cache_values.dims != (hkv, cap, kdh):
        raise ValueError("decode cache must be [num_kv_heads, capacity, kv_head_dim]")
    if update_starts.dims != (3,) or query_start.dims != (1,):
        raise ValueError("update_starts must be si32[3] and query_start si32[1]")

    q_slice = qkv.slice([0, 0], [seq, qp])
    k_slice = qkv.slice([0, qp], [seq, kp])
    v_slice = qkv.slice([0, qp + kp], [seq, kp])
    q_heads = q_slice.reshape([hq, seq, dh])
    new_k = k_slice.reshape([hkv, seq, kdh])
    new_v = v_slice.reshape([hkv, seq, kdh])
    sizes = [hkv, seq, kdh]
    k_cache = cache_keys.dynamic_update_slice(new_k, update_starts, sizes)
    v_cache = cache_values.dynamic_update_slice(new_v, update_starts, sizes)
    k_prefix = k_cache.slice([0, 0, 0], [hkv, cap, kdh])
    v_prefix = v_cache.slice([0, 0, 0], [hkv, cap, kdh])
    k_grouped = _group_kv(k_prefix, hkv, group, hq, cap, kdh)
    v_grouped = _group_kv(v_prefix, hkv, group, hq, cap, kdh)
    scores = q_heads.dot_general(k_grouped, [0], [2], [2])
    scale = fb.scalar_broadcast(float(np.float32(1.0) / np.sqrt(np.float32(dh))), [hq, seq, cap], qkv.dtype)
    scaled = scores * scale
    positions = fb.iota([cap], 0)
    query_pos = positions.dynamic_slice(query_start, [1]).broadcast_to([cap])
    allowed = query_pos.greater_equal(positions)
    zero = fb.scalar_broadcast(0.0, [cap], qkv.dtype)
    neg_large = fb.scalar_broadcast(-1e9, [cap], qkv.dtype)
    base_mask = Tensor.select(allowed, zero, neg_large)
    mask = base_mask.broadcast_to([seq, cap]).broadcast_to([hq, seq, cap])
    masked = scaled + mask
    probs = softmax_last_axis(masked, 2)
    context = probs.dot_general(v_grouped, [0], [2], [1])
    context_out = context.reshape([seq, qp])
    return context_out, k_cache, v_cache


def dynamic_update_slice_into(base: Tensor, update: Tensor, starts: Tensor) -> Tensor:
    """ops/functional/attention.rs:597-646."""
    if starts.dtype != "Si32" or starts.dims != (base.spec.rank,):
        raise ValueError("dynamic_update_slice_into starts must be si32[rank]")
    if len(update.dims) != len(base.dims) or any(u > b for u, b in zip(update.dims, base.dims)):
        raise ValueError("dynamic_update_slice_into update exceeds base")
    return base.dynamic_update_slice(update, starts, list(update.dims))
