""".cyb / .model container: reader and writer for quantised weights.

The container format is the reference's frozen three-rule spec
(/root/reference/reference/format.md:14-20): TOML frontmatter until the first
`~~~`; `~~~name` + LF separates every file inside (:33-35, :58-74); binary files
carry `size` in the frontmatter, text files run to the next `~~~` (:78-84);
text before binary, order = order of `[[files]]` (:110-117).  A .model file is
a .cyb file (/root/reference/reference/cyb-registry.md:14-19).  The writer below
emits the same byte sequence as the reference's in-tree writer does for its own
snapshot (/root/reference/shell/src/worlds/snapshot.rs:71-103): frontmatter,
`~~~config\\n<config>`, then each further part behind its delimiter.

What the tree does NOT pin is the record format of the tensor index ("config,
graph IR, tensor index, tensor data" - /root/reference/decide/pipeline.md:28).
This build defines one: a text part `tensors` (TOML, an array of `[[tensor]]`
tables: name, kind q4|q8, layout block_aos|planar, shape [N,K], offset, nbytes,
and scales_offset / scales_nbytes for planar) pointing into one binary part
`weights`.  Tensor names are HF-canonical (/root/reference/decide/pipeline.md:30).
"""
from __future__ import annotations

import mmap
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np

from . import formats

try:
    import tomllib as _toml          # Python >= 3.11
except ModuleNotFoundError:          # pragma: no cover
    import tomli as _toml

DELIM = b"~~~"


class ContainerError(ValueError):
    pass


@dataclass
class TensorRecord:
    name: str
    kind: str              # "q4" | "q8"
    layout: str            # "block_aos" | "planar"
    shape: Tuple[int, int]  # (N, K)
    offset: int
    nbytes: int
    scales_offset: int = 0
    scales_nbytes: int = 0

    @property
    def bits(self) -> int:
        return {"q4": formats.Q4, "q8": formats.Q8}[self.kind]

    @property
    def layout_code(self) -> int:
        return {"planar": formats.PLANAR, "block_aos": formats.BLOCK_AOS}[self.layout]


def _toml_str(s: str) -> str:
    return '"' + s.replace("\\", "\\\\").replace('"', '\\"') + '"'


def tensor_entry(name: str, q: np.ndarray, scales: np.ndarray, bits: int, layout: int):
    """Canonical (q int8 [N,K], scales u16 [N,K/32]) -> one entry for write_container."""
    N, K = q.shape
    if layout == formats.BLOCK_AOS:
        return {"name": name, "bits": bits, "layout": "block_aos", "shape": (N, K),
                "payload": formats.pack_blocks(q, scales, bits).tobytes(), "scales": b""}
    return {"name": name, "bits": bits, "layout": "planar", "shape": (N, K),
            "payload": formats.pack_planar(q, bits).tobytes(),
            "scales": np.ascontiguousarray(scales, dtype=np.uint16).tobytes()}


def write_container(path: str, model_name: str, config_toml: str, entries: List[dict]) -> None:
    if any(line.startswith("~~~") for line in config_toml.split("\n")):
        raise ContainerError("a text part may not contain a line starting with ~~~")
    if config_toml and not config_toml.endswith("\n"):
        config_toml += "\n"
    blob = bytearray()
    index = []
    for e in entries:
        while len(blob) % 256:               # keep every tensor 256-byte aligned inside the part
            blob.append(0)
        off = len(blob)
        blob += e["payload"]
        rec = [f"[[tensor]]", f"name = {_toml_str(e['name'])}", f"kind = \"q{e['bits']}\"",
               f"layout = \"{e['layout']}\"", f"shape = [{e['shape'][0]}, {e['shape'][1]}]",
               f"offset = {off}", f"nbytes = {len(e['payload'])}"]
        if e["layout"] == "planar":
            while len(blob) % 256:
                blob.append(0)
            rec += [f"scales_offset = {len(blob)}", f"scales_nbytes = {len(e['scales'])}"]
            blob += e["scales"]
        index.append("\n".join(rec) + "\n")
    tensors_toml = "\n".join(index)
    front = (
        "[cyb]\n"
        "types = [\"model\"]\n"
        f"name = {_toml_str(model_name)}\n"
        "\n"
        "[[files]]\nname = \"config\"\nformat = \"toml\"\n"
        "\n"
        "[[files]]\nname = \"tensors\"\nformat = \"toml\"\n"
        "\n"
        "[[files]]\nname = \"weights\"\nformat = \"cybq\"\n"
        f"size = {len(blob)}\n"
    )
    with open(path, "wb") as f:
        f.write(front.encode("utf-8"))
        f.write(b"~~~config\n" + config_toml.encode("utf-8"))
        f.write(b"~~~tensors\n" + tensors_toml.encode("utf-8"))
        f.write(b"~~~weights\n")
        f.write(bytes(blob))


class Container:
    """A parsed container over an mmap of the file (the reference maps its .model
    files too - /root/reference/shell/src/lib.rs:31-33)."""

    def __init__(self, path: str):
        self.path = path
        self._f = open(path, "rb")
        size = os.fstat(self._f.fileno()).st_size
        if size == 0:
            raise ContainerError("empty file")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        self.parts: Dict[str, Tuple[int, int]] = {}     # name -> (offset, length)
        self._parse()

    def close(self) -> None:
        try:
            self._mm.close()
        except BufferError:
            pass                     # numpy views from payload() are still alive; unmapped when they go
        self._f.close()

    # rule 1: TOML frontmatter until the first ~~~ at the start of a line
    def _find_delim(self, start: int) -> int:
        mm = self._mm
        pos = start
        while True:
            i = mm.find(DELIM, pos)
            if i < 0:
                return -1
            if i == 0 or mm[i - 1:i] == b"\n":
                return i
            pos = i + 1

    def _parse(self) -> None:
        mm = self._mm
        first = self._find_delim(0)
        if first < 0:
            raise ContainerError("no ~~~ delimiter: not a .cyb container")
        try:
            self.front = _toml.loads(mm[:first].decode("utf-8"))
        except Exception as e:       # noqa: BLE001 - any TOML error is a container error
            raise ContainerError(f"bad frontmatter: {e}") from e
        files = self.front.get("files", [])
        if not isinstance(files, list) or not files:
            raise ContainerError("frontmatter lists no [[files]]")
        pos = first
        seen_binary = False
        for idx, ent in enumerate(files):
            name = ent.get("name")
            if not isinstance(name, str):
                raise ContainerError("a [[files]] entry has no name")
            # rule 2: the delimiter is `~~~name` followed by LF (CRLF is not a delimiter)
            head = DELIM + name.encode("utf-8") + b"\n"
            if mm[pos:pos + len(head)] != head:
                raise ContainerError(f"expected delimiter ~~~{name} at byte {pos}")
            body = pos + len(head)
            if "size" in ent:           # rule 3: binary parts carry their size
                seen_binary = True
                n = int(ent["size"])
                if n < 0 or body + n > len(mm):
                    raise ContainerError(f"part {name!r}: size {n} runs past the end of the file")
                self.parts[name] = (body, n)
                pos = body + n
            else:
                if seen_binary:
                    # text goes before binary; the one exception the spec draws is a last part without
                    # a size, which simply runs to the end of the file
                    # (/root/reference/reference/format.md:24-31, "binary file (until EOF)")
                    if idx != len(files) - 1:
                        raise ContainerError(f"text part {name!r} after a binary part")
                    self.parts[name] = (body, len(mm) - body)
                    pos = len(mm)
                    continue
                nxt = self._find_delim(body)
                end = nxt if nxt >= 0 else len(mm)
                self.parts[name] = (body, end - body)
                pos = end
        self.name = self.front.get("cyb", {}).get("name", "")

    def text(self, part: str) -> str:
        off, n = self.parts[part]
        return self._mm[off:off + n].decode("utf-8")

    def view(self, part: str) -> memoryview:
        off, n = self.parts[part]
        return memoryview(self._mm)[off:off + n]

    def tensors(self) -> List[TensorRecord]:
        if "tensors" not in self.parts or "weights" not in self.parts:
            raise ContainerError("container has no tensors / weights parts")
        try:
            doc = _toml.loads(self.text("tensors"))
        except Exception as e:       # noqa: BLE001
            raise ContainerError(f"bad tensor index: {e}") from e
        wlen = self.parts["weights"][1]
        out = []
        for t in doc.get("tensor", []):
            try:
                rec = TensorRecord(t["name"], t["kind"], t["layout"], (int(t["shape"][0]), int(t["shape"][1])),
                                   int(t["offset"]), int(t["nbytes"]), int(t.get("scales_offset", 0)),
                                   int(t.get("scales_nbytes", 0)))
            except (KeyError, IndexError, TypeError) as e:
                raise ContainerError(f"bad tensor record: {e}") from e
            if rec.kind not in ("q4", "q8") or rec.layout not in ("planar", "block_aos"):
                raise ContainerError(f"tensor {rec.name!r}: unknown kind/layout")
            N, K = rec.shape
            if K % formats.GROUP or N < 1:
                raise ContainerError(f"tensor {rec.name!r}: bad shape")
            groups = N * (K // formats.GROUP)
            want = groups * (18 if rec.bits == 4 else 34) if rec.layout == "block_aos" else N * K * rec.bits // 8
            if rec.nbytes != want or rec.offset + rec.nbytes > wlen:
                raise ContainerError(f"tensor {rec.name!r}: payload size/offset do not fit")
            if rec.layout == "planar" and (rec.scales_nbytes != groups * 2 or rec.scales_offset + rec.scales_nbytes > wlen):
                raise ContainerError(f"tensor {rec.name!r}: scale plane does not fit")
            out.append(rec)
        return out

    def payload(self, rec: TensorRecord):
        """(q buffer, scales buffer or None) as zero-copy numpy views into the mapping."""
        w = np.frombuffer(self.view("weights"), dtype=np.uint8)
        q = w[rec.offset:rec.offset + rec.nbytes]
        if rec.layout == "planar":
            s = w[rec.scales_offset:rec.scales_offset + rec.scales_nbytes].view(np.uint16)
            return q, s
        return q, None


def load_into(backend, path: str) -> List[TensorRecord]:
    """Uploads every quantised tensor of a container into `backend.weights` by name."""
    c = Container(path)
    try:
        recs = c.tensors()
        for r in recs:
            q, s = c.payload(r)
            backend.upload(r.bits, r.layout_code, r.shape[0], r.shape[1], q, s, name=r.name)
        return recs
    finally:
        c.close()
