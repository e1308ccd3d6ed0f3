"""Writes tests/golden/q38_header_offsets.json: where the fields of the four Qwen3.8 M3 image
headers lie, taken from the reference's own header files by compiling a few lines of C
against them (offsetof / sizeof), so that the loader's restated offsets are checked against
the structs the reference's packer and runtime share
(models/qwen3.8-27b/targets/apple-m3-pro/qwen38_m3_image.h, qwen38_m3_attention_image.h,
qwen38_m3_global_image.h, qwen38_m3_mtp_image.h).  Run in the build container only (needs
/root/reference and gcc); the JSON it writes is what travels.

    python tests/golden/make_q38_header_offsets.py
"""
import json
import pathlib
import re
import subprocess
import tempfile

REFERENCE = pathlib.Path("/root/reference/models/qwen3.8-27b/targets/apple-m3-pro")
HEADERS = {
    "layer": ("qwen38_m3_image.h", "qwen38_m3_image_header", "QWEN38_M3_IMAGE_MAGIC"),
    "attention": ("qwen38_m3_attention_image.h", "qwen38_m3_attention_image_header",
                  "QWEN38_M3_ATTENTION_IMAGE_MAGIC"),
    "global": ("qwen38_m3_global_image.h", "qwen38_m3_global_image_header", "QWEN38_M3_GLOBAL_IMAGE_MAGIC"),
    "mtp": ("qwen38_m3_mtp_image.h", "qwen38_m3_mtp_image_header", "QWEN38_M3_MTP_IMAGE_MAGIC"),
}


def fields_of(header: str, struct: str):
    text = (REFERENCE / header).read_text()
    body = text[text.index("typedef struct {"):text.index("} " + struct + ";")]
    names = []
    for line in body.splitlines():
        match = re.match(r"\s*(?:unsigned char|char|uint32_t|uint64_t|float)\s+(\w+)(\[[^;]*)?;", line)
        if match and not match.group(1).startswith("reserved") and "alignment" not in match.group(1):
            names.append(match.group(1))
    return names


def main():
    program = ["#include <stddef.h>", "#include <stdio.h>"]
    program += [f'#include "{header}"' for header, _, _ in HEADERS.values()]
    program.append("int main(void) {")
    for kind, (header, struct, magic) in HEADERS.items():
        program.append(f'printf("{kind} __size__ %zu %zu\\n", sizeof({struct}), sizeof({struct}));')
        program.append(f'printf("{kind} __magic__ %d %d %d %d %d %d %d %d\\n", {magic}[0], {magic}[1], {magic}[2], '
                       f'{magic}[3], {magic}[4], {magic}[5], {magic}[6], {magic}[7]);')
        for name in fields_of(header, struct):
            program.append(f'printf("{kind} {name} %zu %zu\\n", offsetof({struct}, {name}), '
                           f'sizeof((({struct} *)0)->{name}));')
    program += ["return 0;", "}"]
    with tempfile.TemporaryDirectory() as scratch:
        source = pathlib.Path(scratch) / "offsets.c"
        source.write_text("\n".join(program))
        binary = pathlib.Path(scratch) / "offsets"
        subprocess.run(["gcc", "-std=c11", "-I", str(REFERENCE), str(source), "-o", str(binary)], check=True)
        lines = subprocess.run([str(binary)], check=True, capture_output=True, text=True).stdout.splitlines()
    result = {kind: {"fields": {}} for kind in HEADERS}
    for line in lines:
        kind, name, *numbers = line.split()
        if name == "__size__":
            result[kind]["header_bytes"] = int(numbers[0])
        elif name == "__magic__":
            result[kind]["magic"] = [int(n) for n in numbers]
        else:
            result[kind]["fields"][name] = {"offset": int(numbers[0]), "bytes": int(numbers[1])}
    out = pathlib.Path(__file__).with_name("q38_header_offsets.json")
    out.write_text(json.dumps(result, indent=1, sort_keys=True) + "\n")
    print(out, {kind: len(v["fields"]) for kind, v in result.items()})


if __name__ == "__main__":
    main()
