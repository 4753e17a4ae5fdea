"""Writes tests/golden/vectors.json: small input/output vectors for the checksum, the
digest and the cast, produced WITHOUT the oracle (oracle/) and without the product:

* safe_checksum   a big-integer loop written from the formula of the reference's
                  modelexpress/tensor_utils.py:39-42;
* tensor_digest   a big-integer loop written from refit/reshard/verify.py:112-155 and
                  hashlib.blake2b, the library the reference calls;
* cast            torch's CPU float32 -> bfloat16 conversion (non-NaN inputs only: the NaN
                  image depends on the host's instruction set), and its float32 -> float16,
                  bfloat16 -> float32 and float16 -> float32 conversions (the widening ones on
                  every 64th 16-bit pattern plus the special ones), and float8_e4m3fn -> bfloat16
                  on all 256 codes.

Inputs come from a fixed linear congruential generator so the file is reproducible with
nothing but the standard library and torch.  Run: python tests/golden/make_vectors.py
"""

import hashlib
import json
import struct
from pathlib import Path

import torch

K = 2654435761
M32 = (1 << 32) - 1
M64 = (1 << 64) - 1


def lcg_bytes(seed: int, n: int) -> bytes:
    out = bytearray()
    x = seed & M64
    while len(out) < n:
        x = (x * 6364136223846793005 + 1442695040888963407) & M64
        out += struct.pack("<Q", x)
    return bytes(out[:n])


def checksum(raw: bytes) -> str:
    total = 0
    for i, b in enumerate(raw):
        total += (b * ((i * K + 1) & M32)) & M32
    return format(total & M32, "08x")


def digest(raw: bytes):
    n = len(raw)
    body = n - n % 4
    words = [struct.unpack_from("<i", raw, 4 * k)[0] for k in range(body // 4)]
    rows = len(words) // 1024
    scalars = [n]
    if rows:
        rs = [sum(words[r * 1024:(r + 1) * 1024]) for r in range(rows)]
        scalars += [sum(rs), sum(v * (r + 1) for r, v in enumerate(rs))]
    tail = words[rows * 1024:]
    if tail:
        scalars += [sum(tail), sum(v * (k + 1) for k, v in enumerate(tail))]
    if n % 4:
        scalars += [sum(raw[body:]), n % 4]
    h = hashlib.blake2b(digest_size=16)
    for v in scalars:
        h.update((v & M64).to_bytes(8, "little"))
    return [v & M64 for v in scalars], h.hexdigest()


def main():
    vec = {"checksum": [], "digest": [], "cast": []}
    for seed, n in [(1, 0), (2, 1), (3, 2), (4, 15), (5, 16), (6, 17), (7, 255), (8, 1000), (9, 4096), (10, 4097),
                    (11, 8191), (12, 12288), (13, 20483)]:
        raw = lcg_bytes(seed, n)
        vec["checksum"].append({"seed": seed, "n": n, "hex": raw.hex() if n <= 64 else None, "checksum": checksum(raw)})
        sc, hx = digest(raw)
        vec["digest"].append({"seed": seed, "n": n, "scalars": [str(v) for v in sc], "digest": hx})
    raw = lcg_bytes(99, 4 * 4096)
    bits = [struct.unpack_from("<I", raw, 4 * k)[0] for k in range(4096)]
    extra = [0x00000000, 0x80000000, 0x00000001, 0x00007FFF, 0x00008000, 0x00008001, 0x00018000, 0x3F808000,
             0x3F818000, 0x7F7FFFFF, 0xFF7FFFFF, 0x7F800000, 0xFF800000, 0x7F7F8000, 0x007FFFFF, 0x00800000]
    bits = [b for b in bits + extra if (b & 0x7FFFFFFF) <= 0x7F800000]
    t = torch.tensor([b - (1 << 32) if b >= (1 << 31) else b for b in bits], dtype=torch.int32).view(torch.float32)
    out = t.to(torch.bfloat16).view(torch.int16).tolist()
    vec["cast"] = {"f32_bits": bits, "bf16_bits": [v & 0xFFFF for v in out]}
    extra16 = [0x33000000, 0x33000001, 0x337FFFFF, 0x33800000, 0x387FC000, 0x387FE000, 0x38800000, 0x477FE000,
               0x477FEFFF, 0x477FF000, 0x47800000, 0xC77FF000, 0x3F801000, 0x3F803000, 0x3F801001]
    bits16 = [b for b in bits + extra16 if (b & 0x7FFFFFFF) <= 0x7F800000]
    t = torch.tensor([b - (1 << 32) if b >= (1 << 31) else b for b in bits16], dtype=torch.int32).view(torch.float32)
    vec["cast_f32_f16"] = {"f32_bits": bits16, "f16_bits": [v & 0xFFFF for v in t.to(torch.float16).view(torch.int16).tolist()]}
    halves = sorted(set(list(range(0, 1 << 16, 64)) + [0x0001, 0x03FF, 0x0400, 0x7BFF, 0x7C00, 0xFC00, 0x8001, 0x83FF,
                                                       0x3C00, 0x3F80, 0x7F80, 0xFF80, 0x7F7F, 0x0080, 0x007F]))
    h = torch.tensor([v - (1 << 16) if v >= (1 << 15) else v for v in halves], dtype=torch.int16)
    not_nan16 = [i for i, v in enumerate(halves) if (v & 0x7FFF) <= 0x7C00]
    not_nan_bf = [i for i, v in enumerate(halves) if (v & 0x7FFF) <= 0x7F80]
    f = h.view(torch.float16).to(torch.float32).view(torch.int32).tolist()
    g = h.view(torch.bfloat16).to(torch.float32).view(torch.int32).tolist()
    vec["cast_f16_f32"] = {"f16_bits": [halves[i] for i in not_nan16], "f32_bits": [f[i] & M32 for i in not_nan16]}
    vec["cast_bf16_f32"] = {"bf16_bits": [halves[i] for i in not_nan_bf], "f32_bits": [g[i] & M32 for i in not_nan_bf]}
    vec["cast_f16_bf16"] = {"f16_bits": [halves[i] for i in not_nan16],
                            "bf16_bits": [h.view(torch.float16).to(torch.bfloat16).view(torch.int16).tolist()[i] & 0xFFFF for i in not_nan16]}
    vec["cast_bf16_f16"] = {"bf16_bits": [halves[i] for i in not_nan_bf],
                            "f16_bits": [h.view(torch.bfloat16).to(torch.float16).view(torch.int16).tolist()[i] & 0xFFFF for i in not_nan_bf]}
    codes = torch.arange(256, dtype=torch.uint8)
    vec["cast_f8e4m3_bf16"] = {"f8_bits": list(range(256)),
                               "bf16_bits": [v & 0xFFFF for v in codes.view(torch.float8_e4m3fn).to(torch.bfloat16).view(torch.int16).tolist()]}
    Path(__file__).with_name("vectors.json").write_text(json.dumps(vec, indent=0, separators=(",", ":")))
    print("wrote", Path(__file__).with_name("vectors.json"))


if __name__ == "__main__":
    main()
