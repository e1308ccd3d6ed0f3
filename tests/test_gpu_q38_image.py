"""GPU: the Qwen3.8 image loader (mi355q_q38_image_open) on synthetic images of the four kinds.

No real image exists offline (they are packed from the 27B checkpoint), so the test writes
images itself: a 4096-byte header filled at the offsets of the reference's own structs
(tests/golden/q38_header_offsets.json, produced from the reference's header files) and
code / metadata planes from the library's seeded affine quantizer, at small sizes.  Each
linear the loader returns must have the header's shape and reproduce the oracle on the same
planes; malformed headers must be refused with status 2."""
import json
import pathlib

import numpy as np
import pytest

from conftest import q4_relative_error

pytestmark = pytest.mark.gpu

GOLDEN = json.loads((pathlib.Path(__file__).parent / "golden" / "q38_header_offsets.json").read_text())


def put(header, kind, name, value):
    field = GOLDEN[kind]["fields"][name]
    header[field["offset"]:field["offset"] + field["bytes"]] = np.frombuffer(
        int(value).to_bytes(field["bytes"], "little"), dtype=np.uint8)


def build_image(engine, kind, scalars, linears, version):
    """linears: [(prefix, N, K, seed)] -> (image bytes, {prefix: (quants, meta, N, K)})."""
    header = np.zeros(4096, dtype=np.uint8)
    header[:8] = GOLDEN[kind]["magic"]
    put(header, kind, "version", version)
    put(header, kind, "header_bytes", 4096)
    put(header, kind, "group_size", 64)
    for name, value in scalars.items():
        put(header, kind, name, value)
    planes, parts, offset = {}, [], 4096
    for prefix, N, K, seed in linears:
        quants, meta, _ = engine.synth_q4_affine(seed, 0.02, N, K, engine.META_F16_INTERLEAVED)
        planes[prefix] = (quants, meta, N, K)
        for suffix, data in (("quants", quants.view(np.uint8)), ("metadata", meta.view(np.uint8))):
            put(header, kind, f"{prefix}_{suffix}_offset", offset)
            put(header, kind, f"{prefix}_{suffix}_bytes", data.size)
            parts.append(data.reshape(-1))
            pad = (-data.size) % 4096  # the packer aligns planes to pages
            parts.append(np.zeros(pad, dtype=np.uint8))
            offset += data.size + pad
    return np.concatenate([header] + parts).tobytes(), planes


CASES = {
    "layer": (3, {"hidden_size": 256, "rows": 80, "down_rows": 256, "down_groups_per_row": 2, "layer_index": 5,
                  "delta_input_rows": 48, "delta_input_groups_per_row": 4, "delta_output_rows": 256,
                  "delta_output_groups_per_row": 1},
              [("gate", 80, 256, 1), ("up", 80, 256, 2), ("down", 256, 128, 3), ("delta_input", 48, 256, 4),
               ("delta_output", 256, 64, 5)]),
    "attention": (1, {"hidden_size": 192, "intermediate_size": 64, "layer_index": 3, "input_rows": 100,
                      "input_groups_per_row": 3, "output_rows": 192, "output_groups_per_row": 2},
                  [("gate", 64, 192, 6), ("up", 64, 192, 7), ("down", 192, 64, 8),
                   ("attention_input", 100, 192, 9), ("attention_output", 192, 128, 10)]),
    "global": (1, {"vocab_size": 333, "hidden_size": 128}, [("embedding", 333, 128, 11), ("lm_head", 333, 128, 12)]),
    "mtp": (1, {"hidden_size": 128, "fc_rows": 128, "fc_groups_per_row": 4}, [("fc", 128, 256, 13)]),
}


@pytest.mark.parametrize("kind", list(CASES))
def test_synthetic_image_round_trip(engine, oracle, gpu, kind):
    version, scalars, linears = CASES[kind]
    image_bytes, planes = build_image(engine, kind, scalars, linears, version)
    print(f"q38 image kind={kind} bytes={len(image_bytes)}", flush=True)
    image = gpu.q38_image_open(image_bytes)
    try:
        assert image.kind == kind and image.version == version
        assert image.layer_index == scalars.get("layer_index", 0)
        assert list(image.linears) == [prefix for prefix, *_ in linears]
        for prefix, (quants, meta, N, K) in planes.items():
            weight = image.linears[prefix]
            assert (weight.N, weight.K) == (N, K)
            x = np.stack([engine.synth_normal_f32(50 + m, 1.0, K) for m in range(3)]).astype(np.float16)
            y = gpu.q4_linear(weight, x, engine.F16, engine.F32)
            ref = oracle.q4_linear(quants, meta, None, engine.META_F16_INTERLEAVED, N, K, x, engine.F16, 3)
            assert q4_relative_error(y, ref) <= 1e-3
        if kind == "global":  # the embedding table is used through the row lookup
            quants, meta, N, K = planes["embedding"]
            rows = np.array([0, 332, 17], dtype=np.uint32)
            table = gpu.q4_dequant_rows(image.linears["embedding"], rows)
            expect = oracle.q4_dequantize_rows(quants, meta, None, engine.META_F16_INTERLEAVED, K, rows)
            assert np.array_equal(table.view(np.uint32), expect.view(np.uint32))
    finally:
        image.close()


def test_mlp_only_layer_image(engine, gpu):
    """Version 2 of the layer image holds gate, up and down only."""
    version, scalars, linears = CASES["layer"]
    image_bytes, _ = build_image(engine, "layer", scalars, linears[:3], 2)
    image = gpu.q38_image_open(image_bytes)
    try:
        assert image.version == 2 and list(image.linears) == ["gate", "up", "down"]
    finally:
        image.close()


@pytest.mark.parametrize("damage", ["magic", "version", "header_bytes", "group_size", "bytes", "offset", "short",
                                    "truncated"])
def test_bad_images_are_refused(engine, gpu, damage):
    version, scalars, linears = CASES["mtp"]
    image_bytes, _ = build_image(engine, "mtp", scalars, linears, version)
    data = np.frombuffer(image_bytes, dtype=np.uint8).copy()
    if damage == "magic":
        data[3] ^= 1
    elif damage == "version":
        put(data, "mtp", "version", 9)
    elif damage == "header_bytes":
        put(data, "mtp", "header_bytes", 2048)
    elif damage == "group_size":
        put(data, "mtp", "group_size", 128)
    elif damage == "bytes":
        put(data, "mtp", "fc_quants_bytes", 128 * 256 // 2 + 4)
    elif damage == "offset":
        put(data, "mtp", "fc_metadata_offset", len(image_bytes))
    elif damage == "short":
        data = data[:1000]
    elif damage == "truncated":
        data = data[:len(image_bytes) - 8192]
    with pytest.raises(engine.Mi355qError) as caught:
        gpu.q38_image_open(data.tobytes())
    assert caught.value.status == 2
