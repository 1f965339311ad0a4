#!/usr/bin/env python3
"""Writes the committed container fixtures of this directory (data only; run by hand, never by a test).

spec_example.cyb      the example of the format spec put together: the frontmatter of
                      /root/reference/reference/format.md:40-56 (plus the `program` entry its delimiter
                      example at :62-72 uses, and a trailing `image` part that runs to the end of the
                      file as in the structure sketch at :24-31), the text parts of :62-69 verbatim, and
                      a binary part whose bytes contain a delimiter look-alike and a CRLF.
snapshot_writer.graph the byte sequence the reference's own writer emits
                      (/root/reference/shell/src/worlds/snapshot.rs:71-103): frontmatter with the size of
                      the record blob, `~~~config` + its fixed config text, `~~~cyberlinks` + the records.
                      The record layout is opaque to a container reader; the blob here is 3 x 96 seeded
                      bytes with a `~~~` run inside.
matmul_small.json     known-answer vectors of the operator y = x (scale * q)^T: a 4 x 64 case whose numbers
                      can be followed by hand (scales 1, 0.5, 2, ...; x of small integers), and seeded
                      16 x 96 Q4 and Q8 cases.  q as integers, scales and x as IEEE binary16 bit patterns,
                      expected y from numpy in float64 (no code of this repository's oracle or kernels).
"""
import json
import os
import random

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def spec_example() -> bytes:
    weights = bytes(range(16)) + b"\n~~~config\nnot a delimiter: inside a sized part\r\n" + bytes(range(200, 216))
    image = b"\x89IMG\r\n\x1a\n" + bytes(range(64, 96))
    front = (
        "[cyb]\n"
        "types = [\"model\"]\n"
        "name = \"qwen3-0.6b-abliterated\"\n"
        "\n"
        "[[files]]\n"
        "name = \"config\"\n"
        "format = \"toml\"\n"
        "\n"
        "[[files]]\n"
        "name = \"program\"\n"
        "format = \"text\"\n"
        "\n"
        "[[files]]\n"
        "name = \"weights\"\n"
        "format = \"safetensors\"\n"
        f"size = {len(weights)}\n"
        "\n"
        "[[files]]\n"
        "name = \"image\"\n"
        "format = \"png\"\n"
        "\n"
    )
    body = (
        b"~~~config\n"
        b"architecture = \"Qwen3ForCausalLM\"\n"
        b"hidden_size = 1024\n"
        b"\n"
        b"~~~program\n"
        b"transformer_decoder { layers: 28 }\n"
        b"\n"
        b"~~~weights\n" + weights + b"~~~image\n" + image
    )
    return front.encode("utf-8") + body


def snapshot_writer() -> bytes:
    rng = random.Random(20240607)
    records = bytearray(rng.randrange(256) for _ in range(3 * 96))
    records[100:104] = b"\n~~~"
    front = (
        "[cyb]\n"
        "types = [\"graph\"]\n"
        "name = \"cyb-snapshot\"\n"
        "\n"
        "[[files]]\n"
        "name = \"config\"\n"
        "format = \"toml\"\n"
        "\n"
        "[[files]]\n"
        "name = \"cyberlinks\"\n"
        "format = \"records\"\n"
        f"size = {len(records)}\n"
    )
    config = (
        "chain_id = \"cyb-local\"\n"
        "block = 0\n"
        "\n"
        "[[tokens]]\n"
        "particle = \"0000000000000000000000000000000000000000000000000000000000000000\"\n"
        "weight = 1\n"
    )
    return front.encode() + b"~~~config\n" + config.encode() + b"~~~cyberlinks\n" + bytes(records)


def _f16_bits(a):
    return np.asarray(a, np.float16).view(np.uint16)


def matmul_small() -> str:
    cases = []
    # by hand: row n has q = n+1 in group 0 and -(n+1) in group 1; scales 1 and 0.25; x = 1 in group 0, 2 in group 1:
    # y[n] = 32 (n+1) - 0.25 * 2 * 32 (n+1) = 16 (n+1)
    q = np.zeros((4, 64), np.int64)
    for n in range(4):
        q[n, :32] = n + 1
        q[n, 32:] = -(n + 1)
    sc = np.tile(np.array([1.0, 0.25]), (4, 1))
    x = np.concatenate([np.ones(32), 2 * np.ones(32)])[None, :]
    cases.append(("by_hand_q4", 4, q, sc, x))
    rng = np.random.default_rng(20240607)
    for name, bits, qlo, qhi in (("seeded_q4", 4, -8, 7), ("seeded_q8", 8, -127, 127)):
        q = rng.integers(qlo, qhi + 1, size=(16, 96))
        sc = np.asarray(rng.uniform(0.001, 0.05, size=(16, 3)), np.float16).astype(np.float64)
        x = np.asarray(rng.normal(size=(3, 96)), np.float16).astype(np.float64)
        cases.append((name, bits, q, sc, x))
    out = []
    for name, bits, q, sc, x in cases:
        w = q.astype(np.float64) * np.repeat(sc, 32, axis=1)
        y = x @ w.T
        out.append({"name": name, "bits": bits, "N": int(q.shape[0]), "K": int(q.shape[1]), "M": int(x.shape[0]),
                    "q": q.astype(int).tolist(), "scales_f16_bits": _f16_bits(sc).astype(int).tolist(),
                    "x_f16_bits": _f16_bits(x).astype(int).tolist(), "y": y.tolist()})
    return json.dumps({"operator": "y[m,n] = sum_k x[m,k] * (f32(scale[n,k/32]) * q[n,k])", "cases": out}, separators=(",", ":")) + "\n"


if __name__ == "__main__":
    with open(os.path.join(HERE, "matmul_small.json"), "w") as f:
        f.write(matmul_small())
    for name, data in (("spec_example.cyb", spec_example()), ("snapshot_writer.graph", snapshot_writer())):
        with open(os.path.join(HERE, name), "wb") as f:
            f.write(data)
        print(name, len(data), "bytes")
