"""Shared helpers for the parity tests."""
import numpy as np

Q4, Q8 = 0, 1
FMT_NAME = {Q4: "q4", Q8: "q8"}


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def ref_test_inputs_q4_matmul():
    """Closed-form inputs of the reference's q4_matmul_correctness (tests/gpu_smoke.rs:2683-2712)."""
    m, k, n = 6, 1024, 2048
    i = np.arange(m * k)
    a = (((i % 7).astype(np.float32) - np.float32(3)) * np.float32(0.5)).reshape(m, k)
    i = np.arange(k * n)
    b = ((i % 11).astype(np.float32) - np.float32(5)) * np.float32(0.3)
    b = np.where(i % 1000 == 0, b * np.float32(5), b).astype(np.float32).reshape(k, n)
    return a, b


def golden_ratio_weights(count):
    """make_weights of the reference's q4_layer_nan_hunt (tests/gpu_smoke.rs:2787-2794)."""
    x = (np.arange(count, dtype=np.float64) * 0.618033988) % 1.0
    return ((x * 2.0 - 1.0).astype(np.float32) * np.float32(0.5)).astype(np.float32)


def gemv_parity_inputs(k, n, seed):
    """Inputs of the reference's GEMV parity tests (tests/gemv_parity.rs:74-82)."""
    i = np.arange(k, dtype=np.uint32)
    a = np.sin((i ^ np.uint32(seed)).astype(np.float32) * np.float32(0.003)).astype(np.float32)
    j = np.arange(k * n, dtype=np.uint32)
    s31 = np.uint32((seed * 31) & 0xFFFFFFFF)
    b = np.cos((j ^ s31).astype(np.float32) * np.float32(0.0007)).astype(np.float32)
    return a.reshape(1, k), b.reshape(k, n)


def golden_vectors():
    """Known-answer vectors of tests/golden/known_answers.json: (name, fmt, input [rows, cols] f32, entry)."""
    import json
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "known_answers.json")
    with open(path) as f:
        data = json.load(f)
    out = []
    for v in data["vectors"]:
        w = np.array(v["input_f32_bits"], np.uint32).view(np.float32).reshape(v["rows"], v["cols"])
        out.append((v["name"], Q4 if v["fmt"] == "q4" else Q8, w, v))
    return out, data["f16"]


def check_golden_packed(name, packed, entry):
    """Compare packed bytes with a golden entry (whole bytes, or the prefix + named nibbles)."""
    packed = np.asarray(packed, np.uint8)
    if "packed_hex" in entry:
        assert packed.tobytes().hex() == entry["packed_hex"], name
    else:
        prefix = bytes.fromhex(entry["packed_prefix_hex"])
        assert packed[:len(prefix)].tobytes() == prefix, name
        for idx, nib in entry["nibbles"].items():
            i = int(idx)
            byte = int(packed[4 + i // 2])
            assert ((byte >> 4) if i % 2 else (byte & 0xF)) == nib, (name, i)
