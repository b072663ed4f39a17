"""Writes rope_kats.json: rotary position embedding worked out element by element in double precision from the published
definitions of the scaling rules (linear position interpolation, dynamic NTK, YaRN, LongRoPE, Llama 3), independently of the
vectorised fp32 oracle that the tests hold against it.  Inputs are small seeded tensors [B, H, S, D] (or [T, H, D] for packed
tokens with explicit positions).  Run from the repository root: python tests/golden/make_rope_kats.py"""
import json
import math
import os
import random


def inv_freq(j, rot, o, seq_len):
    kind, base, factor, orig = o.get("scaling_kind", "none"), o.get("base", 10000.0), o.get("scaling_factor", 1.0), o.get("original_max_position_embeddings", 0)
    plain = base ** (-2.0 * j / rot)
    if kind in ("none", "linear"):
        return plain
    if kind == "dynamic_ntk":
        if seq_len > orig and rot > 2:
            base = base * ((factor * seq_len / orig) - (factor - 1.0)) ** (rot / (rot - 2.0))
        return base ** (-2.0 * j / rot)
    if kind == "yarn":
        def correction_dim(rotations):
            return rot * math.log(orig / (rotations * 2.0 * math.pi)) / (2.0 * math.log(base))
        low = max(math.floor(correction_dim(o.get("yarn_beta_fast", 32.0))), 0)
        high = min(math.ceil(correction_dim(o.get("yarn_beta_slow", 1.0))), rot - 1)
        if low == high:
            high += 0.001
        ramp = min(max((j - low) / (high - low), 0.0), 1.0)
        return (plain / factor) * ramp + plain * (1.0 - ramp)
    if kind == "longrope":
        stretch = (o["long_rope_long_factors"] if seq_len > orig else o["long_rope_short_factors"])[j]
        return plain / stretch
    if kind == "llama3":
        low_f, high_f = o.get("llama3_low_freq_factor", 1.0), o.get("llama3_high_freq_factor", 4.0)
        wavelength = 2.0 * math.pi / plain
        if wavelength > orig / low_f:
            return plain / factor
        if wavelength < orig / high_f:
            return plain
        smooth = (orig / wavelength - low_f) / (high_f - low_f)
        return (1.0 - smooth) * plain / factor + smooth * plain
    raise ValueError(kind)


def magnitude(o):
    if o.get("attention_factor") is not None:
        return o["attention_factor"]
    kind, factor = o.get("scaling_kind", "none"), o.get("scaling_factor", 1.0)
    if kind == "yarn" and factor > 1.0:
        return 0.1 * math.log(factor) + 1.0
    if kind == "longrope" and factor > 1.0:
        return math.sqrt(1.0 + math.log(factor) / math.log(o["original_max_position_embeddings"]))
    return 1.0


def rotate(x, shape, o, position_ids=None, effective_length=None):
    """x: flat list in row-major order of `shape`; sequence / head-dimension axes from the options."""
    seq_axis, dim_axis = o.get("sequence_axis", 2), o.get("head_dim_axis", 3)
    strides = [1] * len(shape)
    for a in range(len(shape) - 2, -1, -1):
        strides[a] = strides[a + 1] * shape[a + 1]
    head_dim, seq = shape[dim_axis], shape[seq_axis]
    rot = o.get("rotary_dim", 0) or head_dim
    half = rot // 2
    offset = o.get("position_offset", 0)
    seq_len = max((seq if effective_length is None else effective_length) + max(0, offset), 1.0)
    scale = magnitude(o)
    out = list(x)
    for flat in range(len(x)):
        coords = [(flat // strides[a]) % shape[a] for a in range(len(shape))]
        d, s = coords[dim_axis], coords[seq_axis]
        if d >= rot:
            continue
        if o.get("interleaved", False):
            first, j = d % 2 == 0, d // 2
            peer = flat + strides[dim_axis] if first else flat - strides[dim_axis]
        else:
            first, j = d < half, d % half
            peer = flat + half * strides[dim_axis] if first else flat - half * strides[dim_axis]
        position = float(position_ids[s]) if position_ids is not None else float(s + offset)
        if o.get("scaling_kind", "none") == "linear":
            position /= o["scaling_factor"]
        angle = position * inv_freq(j, rot, o, seq_len)
        sin, cos = math.sin(angle) * scale, math.cos(angle) * scale
        if o.get("inverse", False):
            sin = -sin
        out[flat] = x[flat] * cos - x[peer] * sin if first else x[peer] * sin + x[flat] * cos
    return out


CASES = [
    ("plain", [1, 2, 7, 16], {}),
    ("plain_offset_inverse", [2, 2, 5, 8], {"position_offset": 3, "inverse": True}),
    ("interleaved_partial", [1, 2, 7, 16], {"rotary_dim": 8, "interleaved": True}),
    ("partial_base", [1, 3, 4, 12], {"rotary_dim": 6, "base": 500.0}),
    ("bshd", [2, 5, 3, 8], {"sequence_axis": 1, "head_dim_axis": 3}),
    ("dim_before_sequence", [2, 8, 3, 5], {"sequence_axis": 3, "head_dim_axis": 1, "interleaved": True}),
    ("linear", [1, 2, 7, 16], {"scaling_kind": "linear", "rotary_dim": 8, "scaling_factor": 2.0, "position_offset": 1}),
    ("dynamic_ntk_interleaved", [1, 2, 7, 16],
     {"scaling_kind": "dynamic_ntk", "rotary_dim": 8, "interleaved": True, "scaling_factor": 2.0, "original_max_position_embeddings": 4}),
    ("dynamic_ntk_short", [1, 2, 3, 16], {"scaling_kind": "dynamic_ntk", "rotary_dim": 8, "scaling_factor": 2.0, "original_max_position_embeddings": 4}),
    ("yarn_default_attention_factor", [1, 2, 7, 16],
     {"scaling_kind": "yarn", "rotary_dim": 8, "scaling_factor": 4.0, "original_max_position_embeddings": 16, "yarn_beta_fast": 32.0, "yarn_beta_slow": 1.0}),
    ("yarn_explicit_attention_factor_and_betas", [1, 2, 7, 16],
     {"scaling_kind": "yarn", "rotary_dim": 8, "position_offset": 2, "scaling_factor": 3.0, "original_max_position_embeddings": 12, "attention_factor": 1.25,
      "yarn_beta_fast": 16.0, "yarn_beta_slow": 2.0}),
    ("yarn_wide", [1, 1, 9, 64], {"scaling_kind": "yarn", "scaling_factor": 8.0, "original_max_position_embeddings": 2048}),
    ("longrope_short_factors", [1, 2, 3, 16],
     {"scaling_kind": "longrope", "rotary_dim": 8, "scaling_factor": 4.0, "original_max_position_embeddings": 16,
      "long_rope_short_factors": [1.0, 1.1, 1.2, 1.3], "long_rope_long_factors": [2.0, 2.2, 2.4, 2.6]}),
    ("longrope_long_factors_with_explicit_attention_factor", [1, 2, 7, 16],
     {"scaling_kind": "longrope", "rotary_dim": 8, "position_offset": 3, "scaling_factor": 4.0, "original_max_position_embeddings": 4, "attention_factor": 1.4,
      "long_rope_short_factors": [1.0, 1.1, 1.2, 1.3], "long_rope_long_factors": [2.0, 2.2, 2.4, 2.6]}),
    ("llama3_default_band", [1, 2, 7, 16],
     {"scaling_kind": "llama3", "rotary_dim": 8, "scaling_factor": 8.0, "original_max_position_embeddings": 16, "llama3_low_freq_factor": 1.0,
      "llama3_high_freq_factor": 4.0}),
    ("llama3_custom_band_and_attention_factor", [1, 2, 7, 16],
     {"scaling_kind": "llama3", "rotary_dim": 8, "position_offset": 1, "scaling_factor": 6.0, "original_max_position_embeddings": 12, "attention_factor": 1.1,
      "llama3_low_freq_factor": 1.0, "llama3_high_freq_factor": 3.0}),
    ("llama3_wide", [1, 1, 5, 64], {"scaling_kind": "llama3", "scaling_factor": 8.0, "original_max_position_embeddings": 256, "base": 500000.0}),
]
# explicit positions of packed tokens [T, H, D], and run-time effective lengths
EXTRA = [
    ("packed_position_ids", [9, 2, 8], {"sequence_axis": 0, "head_dim_axis": 2}, [0, 1, 2, 0, 1, 0, 1, 2, 3], None),
    ("dynamic_ntk_effective_length_long", [1, 2, 3, 16],
     {"scaling_kind": "dynamic_ntk", "rotary_dim": 8, "scaling_factor": 2.0, "original_max_position_embeddings": 4}, None, 9),
    ("longrope_effective_length_short", [1, 2, 7, 16],
     {"scaling_kind": "longrope", "rotary_dim": 8, "scaling_factor": 4.0, "original_max_position_embeddings": 4,
      "long_rope_short_factors": [1.0, 1.1, 1.2, 1.3], "long_rope_long_factors": [2.0, 2.2, 2.4, 2.6]}, None, 2),
    ("ids_and_length", [1, 2, 4, 8],
     {"scaling_kind": "dynamic_ntk", "scaling_factor": 3.0, "original_max_position_embeddings": 4, "interleaved": True}, [5, 6, 7, 8], 9),
]


def main():
    rng = random.Random(20240611)
    cases = []
    for name, shape, options, *rest in [c + (None, None) for c in CASES] + EXTRA:
        ids, length = rest[0], rest[1]
        count = 1
        for d in shape:
            count *= d
        # values that fp16 holds exactly, so every storage type starts from the same numbers
        x = [rng.randrange(-2048, 2049) / 1024.0 for _ in range(count)]
        cases.append({"name": name, "shape": shape, "options": options, "position_ids": ids, "effective_sequence_length": length, "x": x,
                      "expected": rotate(x, shape, options, ids, length)})
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rope_kats.json")
    with open(path, "w") as f:
        json.dump({"cases": cases}, f)
    print(path, len(cases), "cases")


if __name__ == "__main__":
    main()
