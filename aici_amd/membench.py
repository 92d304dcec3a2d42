"""The benchmark's yardsticks (csrc/bench/membench.hip, built into libmembench.so): a plain read, a copy, a fill
and a read of shuffled chunks on the device, for holding the decode kernels' bandwidth against what the part
delivers, and a bare stream of MFMAs, for holding the prefill kernels' rate against what the matrix pipes deliver.
Not part of the attention library and not used by it."""
from __future__ import annotations

import ctypes
from pathlib import Path
from typing import Optional

import torch

LIB_PATH = Path(__file__).resolve().parent / "libmembench.so"
_lib = None


def _load():
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise ImportError(f"{LIB_PATH} is not built: run `python -m aici_amd.build`")
        _lib = ctypes.CDLL(str(LIB_PATH))
        _lib.membench_probe.restype = ctypes.c_int
        _lib.membench_probe.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
                                        ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
        _lib.membench_mfma_stream.restype = ctypes.c_int
        _lib.membench_mfma_stream.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    return _lib


MFMA_STREAM_OPERAND_ELEMS = 8 * 512 * 8  # bf16 elements that mfma_stream reads its operands from


def mfma_stream(ops: torch.Tensor, workgroups: int, iters: int) -> float:
    """One launch on torch's current stream of a kernel whose wavefronts (eight per workgroup, two per SIMD) do
    nothing but issue v_mfma_f32_32x32x16_bf16 on the bf16 operands in `ops` (MFMA_STREAM_OPERAND_ELEMS elements);
    returns the flops of the launch."""
    if ops.dtype != torch.bfloat16 or ops.numel() < MFMA_STREAM_OPERAND_ELEMS or not ops.is_contiguous():
        raise ValueError("mfma_stream: ops must be a contiguous bf16 tensor of MFMA_STREAM_OPERAND_ELEMS elements")
    rc = _load().membench_mfma_stream(ops.data_ptr(), None, int(workgroups), int(iters),
                                      ctypes.c_void_p(torch.cuda.current_stream(ops.device).cuda_stream))
    if rc != 0:
        raise RuntimeError(f"membench_mfma_stream failed with code {rc}")
    return float(workgroups) * 8 * iters * 16 * 32768.0


def probe(mode: str, dst: Optional[torch.Tensor], src: Optional[torch.Tensor], chunks: Optional[torch.Tensor] = None,
          chunk_bytes: int = 4096, nontemporal: bool = False) -> None:
    """One launch on torch's current stream: "read" src once, "copy" src to dst, "fill" dst, or "read_chunks":
    the chunks of src (chunk_bytes each) that the int32 tensor `chunks` numbers; `nontemporal`: with the
    hint on every load and store that the data is touched once."""
    modes = {"read": 0, "copy": 1, "fill": 2, "read_chunks": 3}
    t = src if src is not None else dst
    nbytes = t.numel() * t.element_size()
    rc = _load().membench_probe(modes[mode] + (8 if nontemporal else 0), dst.data_ptr() if dst is not None else None,
                                src.data_ptr() if src is not None else None, nbytes,
                                chunks.data_ptr() if chunks is not None else None,
                                chunks.numel() if chunks is not None else 0, int(chunk_bytes),
                                ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream))
    if rc != 0:
        raise RuntimeError(f"membench_probe({mode}) failed with code {rc}" + (" (bad arguments)" if rc == -1 else ""))
