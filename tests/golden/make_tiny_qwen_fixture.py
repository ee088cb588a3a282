"""Extracts a small derived fixture from the reference's committed tiny MLX-4bit model
(crates/forja-host/tests/fixtures/qwen38/{model,reference}.safetensors).

Only data is read: the safetensors container is parsed by hand (8-byte header length, JSON
header, raw little-endian payload); nothing from the reference is imported or executed.
The output pins the MLX nibble order and affine dequantisation:
  hidden_state_0      == dequantised embedding rows of prompt_token_ids (bf16-rounded)
  prompt_last_logits  ~= dequantised lm_head . hidden_state_4[-1]

Run from the repository root with the reference mounted:
  python tests/golden/make_tiny_qwen_fixture.py
"""
import json
import os
import struct

import numpy as np

SOURCE = "/root/reference/crates/forja-host/tests/fixtures/qwen38"
TARGET = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tiny_qwen_mlx4.npz")
NUMPY = {"F32": np.float32, "U32": np.uint32, "I64": np.int64, "BF16": np.uint16}


def read_safetensors(path):
    with open(path, "rb") as handle:
        (header_len,) = struct.unpack("<Q", handle.read(8))
        header = json.loads(handle.read(header_len))
        payload = handle.read()
    tensors = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        begin, end = meta["data_offsets"]
        array = np.frombuffer(payload[begin:end], dtype=NUMPY[meta["dtype"]]).reshape(meta["shape"])
        tensors[name] = array.copy()
    return tensors


def main():
    model = read_safetensors(os.path.join(SOURCE, "model.safetensors"))
    reference = read_safetensors(os.path.join(SOURCE, "reference.safetensors"))
    prefix = "language_model."
    np.savez(
        TARGET,
        embed_packed=model[prefix + "model.embed_tokens.weight"],
        embed_scales_bf16=model[prefix + "model.embed_tokens.scales"],
        embed_biases_bf16=model[prefix + "model.embed_tokens.biases"],
        lm_head_packed=model[prefix + "lm_head.weight"],
        lm_head_scales_bf16=model[prefix + "lm_head.scales"],
        lm_head_biases_bf16=model[prefix + "lm_head.biases"],
        prompt_token_ids=reference["prompt_token_ids"].astype(np.uint32),
        hidden_state_0=reference["hidden_state_0"],
        final_hidden_last=reference["hidden_state_4"][-1],
        prompt_last_logits=reference["prompt_last_logits"],
        first_greedy_token=reference["greedy_token_ids"][:1].astype(np.uint32),
    )
    print("wrote", TARGET, os.path.getsize(TARGET), "bytes")


if __name__ == "__main__":
    main()
