"""Writes tests/golden/rand32.json: known-answer vectors for the counter-based
random stream, produced by a pure-python-integer statement of the hash that is
independent of the numpy (oracle) and HIP (product) implementations."""
import json
import os


def fmix(h):
    h &= 0xFFFFFFFF
    h ^= h >> 16
    h = (h * 0x85EBCA6B) & 0xFFFFFFFF
    h ^= h >> 13
    h = (h * 0xC2B2AE35) & 0xFFFFFFFF
    h ^= h >> 16
    return h


def r32(seed, stream, idx):
    ka = (fmix(seed ^ 0x9E3779B9) + stream * 0x85EBCA77) & 0xFFFFFFFF
    kb = fmix((stream + 0xC2B2AE3D) & 0xFFFFFFFF) ^ seed
    x = (idx + ka) & 0xFFFFFFFF
    x ^= x >> 16
    x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= kb
    x ^= x >> 15
    x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x


if __name__ == "__main__":
    cases = []
    for seed, stream in [(0, 0), (1, 0), (0, 1), (12345, 678), (0xFFFFFFFF, 0xFFFFFFFF)]:
        idx = [0, 1, 2, 3, 255, 65535, 65536, 2 ** 31, 2 ** 32 - 1]
        cases.append({"seed": seed, "stream": stream, "idx": idx,
                      "out": [r32(seed, stream, i) for i in idx]})
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "rand32.json"), "w") as f:
        json.dump({"generator": "tests/golden/make_rand32.py (pure-python integer restatement)",
                   "cases": cases}, f, indent=1)
