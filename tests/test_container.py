"""The .cyb / .model container: the three rules of the reference's format spec
(/root/reference/reference/format.md:14-20) and this build's tensor index."""
import os
import subprocess

import numpy as np
import pytest

from cyb_amd import container, formats, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST_TEST = os.path.join(ROOT, "tests", "cpp", "_build", "host_test")


def _entries():
    w = synth.weights(41, 48, 160)
    q4, s4 = formats.quantize(w, 4)
    q8, s8 = formats.quantize(w[:32], 8)
    return (q4, s4, q8, s8,
            [container.tensor_entry("model.layers.0.mlp.up_proj.weight", q4, s4, 4, formats.BLOCK_AOS),
             container.tensor_entry("model.layers.0.mlp.down_proj.weight", q8, s8, 8, formats.PLANAR),
             container.tensor_entry("model.layers.0.self_attn.q_proj.weight", q4, s4, 4, formats.PLANAR)])


def test_round_trip(tmp_path):
    q4, s4, q8, s8, ents = _entries()
    path = str(tmp_path / "tiny.model")
    container.write_container(path, "tiny", 'architecture = "LlamaForCausalLM"\nhidden_size = 160\n', ents)
    c = container.Container(path)
    assert c.name == "tiny"
    assert list(c.parts) == ["config", "tensors", "weights"]          # order of [[files]]
    assert c.text("config").startswith('architecture = "LlamaForCausalLM"')
    recs = c.tensors()
    assert [r.name for r in recs] == [e["name"] for e in ents]
    r0, r1, r2 = recs
    assert (r0.kind, r0.layout, r0.shape) == ("q4", "block_aos", (48, 160))
    q, s = c.payload(r0)
    qq, ss = formats.unpack_blocks(q, 4, 48, 160)
    assert np.array_equal(qq, q4) and np.array_equal(ss, s4) and s is None
    q, s = c.payload(r1)
    assert np.array_equal(formats.unpack_planar(q, 8, 32, 160), q8) and np.array_equal(s.reshape(32, 5), s8)
    q, s = c.payload(r2)
    assert np.array_equal(formats.unpack_planar(q, 4, 48, 160), q4) and np.array_equal(s.reshape(48, 5), s4)
    assert all(r.offset % 256 == 0 for r in recs)
    c.close()


def test_layout_on_disk_follows_the_three_rules(tmp_path):
    *_, ents = _entries()
    path = str(tmp_path / "t.cyb")
    container.write_container(path, "t", "a = 1\n", ents[:1])
    raw = open(path, "rb").read()
    first = raw.index(b"~~~")
    assert raw[:first].decode().startswith("[cyb]\n")                 # rule 1: frontmatter first
    assert raw[first:first + 10] == b"~~~config\n"                    # rule 2: ~~~name + LF
    assert b"\r" not in raw[:raw.index(b"~~~weights\n")]
    size = int(raw[:first].decode().split("size = ")[1].split("\n")[0])
    assert raw.endswith(raw[-size:]) and len(raw) == raw.index(b"~~~weights\n") + len(b"~~~weights\n") + size   # rule 3


def test_binary_payload_may_contain_delimiter_bytes(tmp_path):
    # bytes of the binary part are never scanned for ~~~ (its size is in the frontmatter)
    q = np.full((16, 32), 7, np.int8)
    s = np.full((16, 1), 0x3C00, np.uint16)
    e = container.tensor_entry("w", q, s, 8, formats.PLANAR)
    e["payload"] = (b"\n~~~tensors\n" + e["payload"])[:len(e["payload"])]
    path = str(tmp_path / "d.model")
    container.write_container(path, "d", "", [e])
    c = container.Container(path)
    assert len(c.tensors()) == 1 and c.parts["weights"][1] >= 16 * 32
    c.close()


@pytest.mark.parametrize("damage", ["no_delim", "crlf", "size_past_end", "text_after_binary", "bad_index", "truncated_payload"])
def test_malformed_containers_are_rejected(tmp_path, damage):
    *_, ents = _entries()
    path = str(tmp_path / "m.model")
    container.write_container(path, "m", "a = 1\n", ents[:1])
    raw = open(path, "rb").read()
    if damage == "no_delim":
        raw = raw.replace(b"~~~", b"---")
    elif damage == "crlf":
        raw = raw.replace(b"~~~config\n", b"~~~config\r\n")
    elif damage == "size_past_end":
        raw = raw[:-100]
    elif damage == "text_after_binary":
        raw = raw.replace(b'[[files]]\nname = "config"\nformat = "toml"\n', b'[[files]]\nname = "config"\nformat = "toml"\nsize = 6\n')
    elif damage == "bad_index":
        raw = raw.replace(b'kind = "q4"', b'kind = "q5"')
    elif damage == "truncated_payload":
        raw = raw.replace(b"nbytes = 4320", b"nbytes = 4319")
    open(path, "wb").write(raw)
    with pytest.raises(container.ContainerError):
        c = container.Container(path)
        c.tensors()
    # the C++ reader agrees
    if os.path.exists(HOST_TEST):
        out = subprocess.run([HOST_TEST, "--parse", path], capture_output=True, text=True)
        assert out.returncode == 1 and out.stdout.startswith("ERROR"), out.stdout


def test_text_part_may_not_hide_a_delimiter(tmp_path):
    *_, ents = _entries()
    with pytest.raises(container.ContainerError):
        container.write_container(str(tmp_path / "x.model"), "x", "a = 1\n~~~weights\n", ents[:1])


def test_cpp_reader_matches_python(tmp_path):
    if not os.path.exists(HOST_TEST):
        pytest.fail("tests/cpp/_build/host_test missing: run __graft_entry__.build()")
    *_, ents = _entries()
    path = str(tmp_path / "tiny.model")
    container.write_container(path, "tiny model", "hidden_size = 160\n", ents)
    out = subprocess.run([HOST_TEST, "--parse", path], capture_output=True, text=True, check=True).stdout.split("\n")
    assert out[0] == "name tiny model"
    c = container.Container(path)
    for line, r in zip(out[1:], c.tensors()):
        assert line == f"tensor {r.name} {r.kind} {r.layout} {r.shape[0]} {r.shape[1]} {r.offset}"
    c.close()


# ---- committed fixtures (tests/golden/, written by tests/golden/make_fixtures.py) -----------------

GOLDEN = os.path.join(ROOT, "tests", "golden")


def _fnv1a(data: bytes) -> str:
    h = 1469598103934665603
    for b in data:
        h = ((h ^ b) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return f"{h:016x}"


def _cpp_parts(path, names):
    out = subprocess.run([HOST_TEST, "--parts", path] + names, capture_output=True, text=True, check=True).stdout.split("\n")
    return out[0], {l.split()[1]: (int(l.split()[2]), l.split()[3]) for l in out[1:] if l.startswith("part ") and "missing" not in l}


def test_fixture_spec_example_is_read_by_both_readers():
    """The format spec's own example (/root/reference/reference/format.md:40-72), assembled into a file."""
    path = os.path.join(GOLDEN, "spec_example.cyb")
    c = container.Container(path)
    assert c.name == "qwen3-0.6b-abliterated"
    assert c.front["cyb"]["types"] == ["model"]
    assert list(c.parts) == ["config", "program", "weights", "image"]           # order of [[files]]
    assert c.text("config") == 'architecture = "Qwen3ForCausalLM"\nhidden_size = 1024\n\n'
    assert c.text("program") == "transformer_decoder { layers: 28 }\n\n"
    w = bytes(c.view("weights"))
    assert len(w) == c.front["files"][2]["size"] and b"\n~~~config\n" in w and b"\r\n" in w     # never scanned
    img = bytes(c.view("image"))
    assert img.startswith(b"\x89IMG\r\n") and len(img) == 40                      # last part: runs to the end of the file
    raw = open(path, "rb").read()
    assert raw.endswith(img)
    with pytest.raises(container.ContainerError):
        c.tensors()                                                              # not a tensor container: said so, not guessed
    if os.path.exists(HOST_TEST):
        name, parts = _cpp_parts(path, ["config", "program", "weights", "image", "nope"])
        assert name == "name qwen3-0.6b-abliterated"
        assert parts == {n: (c.parts[n][1], _fnv1a(bytes(c.view(n)))) for n in ("config", "program", "weights", "image")}
    c.close()


def test_fixture_of_the_reference_writer_is_read_by_both_readers():
    """The byte stream the reference's own .cyb writer emits
    (/root/reference/shell/src/worlds/snapshot.rs:71-103): frontmatter, ~~~config, ~~~cyberlinks + size bytes."""
    path = os.path.join(GOLDEN, "snapshot_writer.graph")
    raw = open(path, "rb").read()
    c = container.Container(path)
    assert c.name == "cyb-snapshot" and c.front["cyb"]["types"] == ["graph"]
    assert [f["format"] for f in c.front["files"]] == ["toml", "records"]
    cfg = c.text("config")
    assert cfg.startswith('chain_id = "cyb-local"\nblock = 0\n') and cfg.endswith("weight = 1\n")
    rec = bytes(c.view("cyberlinks"))
    assert len(rec) == 3 * 96 == c.front["files"][1]["size"] and raw.endswith(rec) and b"\n~~~" in rec
    if os.path.exists(HOST_TEST):
        name, parts = _cpp_parts(path, ["config", "cyberlinks"])
        assert name == "name cyb-snapshot"
        assert parts == {"config": (len(cfg.encode()), _fnv1a(cfg.encode())), "cyberlinks": (len(rec), _fnv1a(rec))}
    c.close()


def test_fixtures_match_their_generator():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert open(os.path.join(GOLDEN, "spec_example.cyb"), "rb").read() == mod.spec_example()
    assert open(os.path.join(GOLDEN, "snapshot_writer.graph"), "rb").read() == mod.snapshot_writer()
