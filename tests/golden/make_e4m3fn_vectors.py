"""Writes the e4m3fn codec fixtures from torch's CPU float8_e4m3fn cast (a
library routine, independent of the oracle).  Run once in the build container:

    python tests/golden/make_e4m3fn_vectors.py

Outputs (committed beside this script):
  e4m3fn_decode_256.f32        256 little-endian f32: value of every byte
  e4m3fn_encode_bf16_65536.u8  byte i = e4m3fn(clamp(bf16 with bit pattern i, +-448));
                               NaN inputs are stored as 0x7f (the reference maps
                               every NaN to 0x7f, mojo/stdlib/std/builtin/simd.mojo:3886-3888)
"""
import os

import numpy as np
import torch

here = os.path.dirname(os.path.abspath(__file__))

dec = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
dec.astype("<f4").tofile(os.path.join(here, "e4m3fn_decode_256.f32"))

bits = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
x = torch.from_numpy(bits.copy())
enc = x.clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy().copy()
enc[np.isnan(bits)] = 0x7F
enc.tofile(os.path.join(here, "e4m3fn_encode_bf16_65536.u8"))
print("wrote", dec.size, "decode values and", enc.size, "encode bytes")
