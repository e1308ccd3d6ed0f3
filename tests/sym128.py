"""Test-side packer for the symmetric group-128 Q4 records (66 bytes: bf16 scale + 64 code
bytes), written from the format description the reference's runtime reads
(qwen35_task.c:286-303, 426-450) and its packer documents (compiler/q4_image.py:120-146):
scale = max(-min/8, max/7) (1 when 0), q = clip(rint(w/scale), -8, 7), two's-complement nibble,
even column in the low nibble.  Only used to make test inputs."""
import numpy as np

from conftest import bf16_bits


def pack_sym128(weights):
    weights = np.asarray(weights, dtype=np.float32)
    rows, cols = weights.shape
    assert cols % 128 == 0
    groups = cols // 128
    blocks = weights.reshape(rows, groups, 128)
    scale = np.maximum(-blocks.min(axis=-1) / np.float32(8.0), blocks.max(axis=-1) / np.float32(7.0))
    scale[scale == 0] = np.float32(1.0)
    q = np.clip(np.rint(blocks / scale[..., None]), -8, 7).astype(np.int8)
    nib = (q.astype(np.int16) & 0xF).astype(np.uint8)
    records = np.empty((rows, groups, 66), dtype=np.uint8)
    records[..., :2] = bf16_bits(scale).view(np.uint8).reshape(rows, groups, 2)
    records[..., 2:] = nib[..., 0::2] | (nib[..., 1::2] << 4)
    return records


def output_block(records, block):
    """[row/block][group][row%block][record]: the permutation the reference's unit test asserts
    (tests/test_q4_output_block.py:24-31: reshape(R/4, 4, G, rec).transpose(0, 2, 1, 3))."""
    rows, groups, size = records.shape
    if rows % block:
        raise ValueError("rows not divisible by the output block")
    return np.ascontiguousarray(
        records.reshape(rows // block, block, groups, size).transpose(0, 2, 1, 3)).reshape(-1)
