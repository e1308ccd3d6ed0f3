"""The image loader's header offsets against the reference's structs (CPU).

tests/golden/q38_header_offsets.json holds offsetof()/sizeof() of every field of the four
Qwen3.8 M3 image headers, produced by compiling against the reference's own header files
(tests/golden/make_q38_header_offsets.py).  The loader reads headers at restated byte
offsets; every field it reads must sit where the reference's struct puts it."""
import json
import pathlib

import pytest

GOLDEN = pathlib.Path(__file__).parent / "golden" / "q38_header_offsets.json"
KINDS = ["layer", "attention", "global", "mtp"]


@pytest.mark.parametrize("kind", range(4))
def test_loader_offsets_match_reference_structs(engine, kind):
    reference = json.loads(GOLDEN.read_text())[KINDS[kind]]
    assert reference["header_bytes"] == 4096
    fields = engine.q38_layout_fields(kind)
    assert engine.library().mi355q_q38_kind_name(kind).decode() == KINDS[kind]
    assert len(fields) >= 11
    for name, (offset, size) in fields.items():
        assert name in reference["fields"], f"{KINDS[kind]}: the reference struct has no field {name}"
        assert (offset, size) == (reference["fields"][name]["offset"], reference["fields"][name]["bytes"]), name
    # every plane descriptor of the reference header is read by the loader
    for name in reference["fields"]:
        if name.endswith(("_quants_offset", "_quants_bytes", "_metadata_offset", "_metadata_bytes")):
            assert name in fields, f"{KINDS[kind]}: loader ignores {name}"


def test_layout_query_past_the_end(engine):
    import ctypes
    name, offset, size = ctypes.c_char_p(), ctypes.c_uint32(), ctypes.c_uint32()
    lib = engine.library()
    assert lib.mi355q_q38_layout_field(0, 10_000, ctypes.byref(name), ctypes.byref(offset), ctypes.byref(size)) == 2
    assert lib.mi355q_q38_layout_field(7, 0, ctypes.byref(name), ctypes.byref(offset), ctypes.byref(size)) == 2
    assert lib.mi355q_q38_kind_name(9) is None
