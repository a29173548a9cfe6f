"""GGUF tensors -> the affine triplet, on the GPU.

Mirror of what ``mx.load("*.gguf")`` does for the quantized tensor types it
keeps quantized (reference: ``mlx/io/gguf.cpp`` ``load_gguf`` / ``load_arrays``
and ``mlx/io/gguf_quants.cpp:102-166``): a ``name.weight`` tensor of GGML type
Q4_0, Q4_1 or Q8_0 becomes ``name.weight`` (uint32 codes), ``name.scales`` and
``name.biases`` (float16, group size 32), ready for ``quantized_matmul`` with
``group_size=32`` and ``bits`` 4 or 8.  F32 / F16 tensors are returned as they
are.  The block shuffle itself is done by the HIP kernel behind
``mlxrocm_gguf_repack``; this module only parses the container (a plain
little-endian header, key/value metadata and a table of tensors, GGUF versions
2 and 3) and moves the bytes to the device.  Other GGML quantized types, which
the reference dequantizes to float16 with gguflib while loading, are rejected.
"""
from __future__ import annotations

import mmap
import struct
from typing import Dict, Tuple

import numpy as np
import torch

from . import _lib

GGML_F32, GGML_F16, GGML_Q4_0, GGML_Q4_1, GGML_Q8_0 = 0, 1, 2, 3, 8
_BLOCK_BYTES = {GGML_Q4_0: 18, GGML_Q4_1: 20, GGML_Q8_0: 34}
_BITS = {GGML_Q4_0: 4, GGML_Q4_1: 4, GGML_Q8_0: 8}
_WEIGHTS_PER_BLOCK = 32

# metadata value types of the GGUF key/value section
_SCALAR = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?",
           10: "<Q", 11: "<q", 12: "<d"}
_STRING, _ARRAY = 8, 9


class _Reader:
    def __init__(self, buf):
        self.buf = buf
        self.pos = 0

    def take(self, fmt: str):
        size = struct.calcsize(fmt)
        if self.pos + size > len(self.buf):
            raise ValueError("[load_gguf] file ends inside the header")
        (v,) = struct.unpack_from(fmt, self.buf, self.pos)
        self.pos += size
        return v

    def string(self) -> str:
        n = self.take("<Q")
        if self.pos + n > len(self.buf):
            raise ValueError("[load_gguf] file ends inside a string")
        s = bytes(self.buf[self.pos:self.pos + n])
        self.pos += n
        return s.decode("utf-8", errors="replace")

    def value(self, vtype: int):
        if vtype in _SCALAR:
            return self.take(_SCALAR[vtype])
        if vtype == _STRING:
            return self.string()
        if vtype == _ARRAY:
            etype = self.take("<I")
            count = self.take("<Q")
            return [self.value(etype) for _ in range(count)]
        raise ValueError(f"[load_gguf] unknown metadata value type {vtype}")


def read_header(buf) -> Tuple[dict, list, int]:
    """Parse the GGUF header of ``buf`` (bytes-like).  Returns (metadata,
    tensors, data_offset); every tensor is (name, shape, ggml_type, offset) with
    the shape in row-major order (GGUF stores dimensions innermost first)."""
    r = _Reader(buf)
    if bytes(buf[:4]) != b"GGUF":
        raise ValueError("[load_gguf] not a GGUF file")
    r.pos = 4
    version = r.take("<I")
    if version not in (2, 3):
        raise ValueError(f"[load_gguf] unsupported GGUF version {version}")
    n_tensors = r.take("<Q")
    n_kv = r.take("<Q")
    metadata = {}
    for _ in range(n_kv):
        key = r.string()
        metadata[key] = r.value(r.take("<I"))
    tensors = []
    for _ in range(n_tensors):
        name = r.string()
        n_dims = r.take("<I")
        dims = [r.take("<Q") for _ in range(n_dims)]
        ggml_type = r.take("<I")
        offset = r.take("<Q")
        tensors.append((name, tuple(reversed(dims)), ggml_type, offset))
    alignment = int(metadata.get("general.alignment", 32))
    data_offset = (r.pos + alignment - 1) // alignment * alignment
    return metadata, tensors, data_offset


def repack(blocks: torch.Tensor, ggml_type: int, shape) -> Tuple[torch.Tensor, ...]:
    """GGML blocks (uint8 tensor on the GPU, the tensor's bytes as stored in the
    file) of a tensor of logical ``shape`` -> (weight, scales, biases)."""
    if ggml_type not in _BLOCK_BYTES:
        raise ValueError(f"[load_gguf] GGML type {ggml_type} is not kept quantized")
    shape = tuple(int(s) for s in shape)
    if not shape or shape[-1] % _WEIGHTS_PER_BLOCK != 0:
        # gguf_quants.cpp:115-120
        raise RuntimeError(
            f"[load_gguf] tensor has incompatible last dim shape: {shape[-1] if shape else 0}"
        )
    if blocks.device.type != "cuda":
        raise RuntimeError(f"[load_gguf] mlx_amd runs on the GPU only; got a tensor on {blocks.device}")
    n_blocks = int(np.prod(shape)) // _WEIGHTS_PER_BLOCK
    blocks = blocks.contiguous().view(torch.uint8).reshape(-1)
    if blocks.numel() != n_blocks * _BLOCK_BYTES[ggml_type]:
        raise ValueError(
            f"[load_gguf] {blocks.numel()} bytes do not hold {n_blocks} blocks of GGML type {ggml_type}"
        )
    if blocks.data_ptr() % 16 != 0:
        blocks = blocks.clone()  # fresh allocations are aligned
    per_word = 32 // _BITS[ggml_type]
    dev = blocks.device
    weight = torch.empty(shape[:-1] + (shape[-1] // per_word,), dtype=torch.uint32, device=dev)
    sb_shape = shape[:-1] + (shape[-1] // _WEIGHTS_PER_BLOCK,)
    scales = torch.empty(sb_shape, dtype=torch.float16, device=dev)
    biases = torch.empty(sb_shape, dtype=torch.float16, device=dev)
    lib = _lib.load()
    _lib.check(
        lib.mlxrocm_gguf_repack(
            blocks.data_ptr(), weight.data_ptr(), scales.data_ptr(), biases.data_ptr(),
            n_blocks, ggml_type, torch.cuda.current_stream(dev).cuda_stream,
        )
    )
    return weight, scales, biases


def load_gguf(path, device="cuda") -> Tuple[Dict[str, torch.Tensor], dict]:
    """Load every tensor of a GGUF file onto ``device``.  Returns (arrays,
    metadata) like ``mx.load(path, return_metadata=True)``."""
    arrays: Dict[str, torch.Tensor] = {}
    with open(path, "rb") as f:
        with mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ) as mm:
            metadata, tensors, data_offset = read_header(mm)
            file_size = len(mm)

        def read(start: int, count: int, np_dtype) -> np.ndarray:
            host = np.empty(count, dtype=np_dtype)
            if start + host.nbytes > file_size:
                raise ValueError("[load_gguf] tensor data runs past the end of the file")
            f.seek(start)
            if f.readinto(memoryview(host).cast("B")) != host.nbytes:
                raise ValueError("[load_gguf] short read")
            return host

        for name, shape, ggml_type, offset in tensors:
            n = int(np.prod(shape)) if shape else 1
            start = data_offset + offset
            if ggml_type in (GGML_F32, GGML_F16):
                np_dtype = np.float32 if ggml_type == GGML_F32 else np.float16
                host = read(start, n, np_dtype).reshape(shape)
                _insert(arrays, name, torch.from_numpy(host).to(device))
            elif ggml_type in _BLOCK_BYTES:
                if not shape or shape[-1] % _WEIGHTS_PER_BLOCK != 0:
                    raise RuntimeError(
                        f"[load_gguf] tensor {name}has incompatible last dim shape: "
                        f"{shape[-1] if shape else 0}"
                    )
                nbytes = n // _WEIGHTS_PER_BLOCK * _BLOCK_BYTES[ggml_type]
                blocks = torch.from_numpy(read(start, nbytes, np.uint8)).to(device)
                weight, scales, biases = repack(blocks, ggml_type, shape)
                _insert(arrays, name, weight)
                # gguf_quants.cpp:160-165: ".weight" is swapped for the suffix
                prefix = name[: len(name) - len(".weight")]
                _insert(arrays, prefix + ".scales", scales)
                _insert(arrays, prefix + ".biases", biases)
            else:
                raise RuntimeError(
                    f"[load_gguf] tensor {name} has GGML type {ggml_type}; only F32, F16, "
                    "Q4_0, Q4_1 and Q8_0 have a ROCm implementation."
                )
    return arrays, metadata


def _insert(arrays: Dict[str, torch.Tensor], name: str, value: torch.Tensor) -> None:
    if name in arrays:
        raise RuntimeError(
            f"[load_gguf] Duplicate parameter name {name} this can happend when loading "
            "quantized tensors."
        )
    arrays[name] = value
