"""Run a `Program` (programs/configs.py) through the PJRT C API of the plugin."""
from __future__ import annotations

from typing import List, Sequence

import numpy as np

from . import pjrt
from .programs.configs import Program, to_device_bytes


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def upload(client: pjrt.Client, arrays: Sequence[np.ndarray], dtypes: Sequence[str]) -> List[pjrt.Buffer]:
    out = []
    for a, d in zip(arrays, dtypes):
        host = to_device_bytes(a, d)
        out.append(client.buffer_from_pyval(host, pjrt.MLIR_TO_PJRT[d]))
    return out


def download(buf: pjrt.Buffer) -> np.ndarray:
    """Host copy of a device buffer; bf16 is widened to float32."""
    raw = buf.to_numpy()
    if buf.dtype_code() == pjrt.BF16:
        return bf16_bits_to_f32(raw)
    return raw


class CompiledProgram:
    def __init__(self, program: Program, client: pjrt.Client = None):
        self.program = program
        self.client = client or pjrt.get_client()
        self.exe = self.client.compile_and_load(program.text)
        self.state = upload(self.client, program.inputs, program.input_dtypes)

    def step(self) -> List[pjrt.Buffer]:
        """One execution; outputs named in `feedback` replace the matching inputs (train-state threading)."""
        outs = self.exe.execute(self.state, donate=True)      # the state inputs are consumed and replaced by the outputs
        for k, i in self.program.feedback.items():
            self.state[i] = outs[k]
        return outs

    def run_once(self) -> List[np.ndarray]:
        return [download(b) for b in self.exe.execute(self.state)]
