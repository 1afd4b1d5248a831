"""Helpers shared by the GPU parity tests: move raw numpy storage to the GPU
and back, and the reference's pass criteria."""
import numpy as np
import torch

from oracle import rock_oracle as orc

TORCH = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16, "i8": torch.int8,
         "fp8": torch.float8_e4m3fn, "bf8": torch.float8_e5m2, "i32": torch.int32}
CODE = orc.TYPE_CODES
_CARRIER = {"f32": np.float32, "f16": np.int16, "bf16": np.int16, "i8": np.int8, "fp8": np.uint8,
            "bf8": np.uint8, "i32": np.int32}

# thresholds of the reference verifier (rocmlir-gen.cpp:2850-2868): RMS 3e-5 for
# f32 results, 1e-3 for 16-bit results; 8-bit float outputs get the 16-bit gate
RMS_THRESHOLD = {"f32": 3e-5, "f16": 1e-3, "bf16": 1e-2, "fp8": 0.1, "bf8": 0.2}


def quantise(values_f32, dtype):
    """f32 values -> (raw numpy storage, the same values widened back to f32)"""
    raw = orc.narrow(np.asarray(values_f32, np.float32), CODE[dtype])
    return raw, orc.widen(raw, CODE[dtype])


def to_gpu(raw, dtype, device):
    t = torch.from_numpy(np.ascontiguousarray(raw).view(_CARRIER[dtype])).to(device)
    return t.view(TORCH[dtype])


def to_f32(t, dtype):
    """GPU tensor of `dtype` -> flat float32 numpy (exact widening)"""
    flat = t.detach().reshape(-1)
    if dtype in ("f32", "i8", "i32"):
        return flat.cpu().numpy().astype(np.float32)
    carrier = torch.int16 if dtype in ("f16", "bf16") else torch.uint8
    raw = flat.view(carrier).cpu().numpy()
    raw = raw.view(np.uint16) if carrier is torch.int16 else raw
    return orc.widen(raw, CODE[dtype])


def check_float(gpu_f32, oracle_f32, out_dtype, rms=None, max_abs=None):
    """The reference's comparison: round the f32 oracle through the output
    type (rocmlir-gen.cpp:2828-2840), then the RMS and max-abs gates.  The
    max-rel metric is reported but not gated: with mixed-sign real data a
    reference value next to zero makes it arbitrarily large (the reference
    warns about exactly this, rocmlir-gen.cpp:2681-2693)."""
    val = orc.round_through(oracle_f32, CODE[out_dtype])
    res = orc.verify_float(gpu_f32, val, thr_rms=rms if rms is not None else RMS_THRESHOLD[out_dtype],
                           thr_abs=max_abs if max_abs is not None else 100.0, thr_rel=1e30)
    assert not np.isnan(gpu_f32).any(), "NaN in GPU result"
    assert res.passed(), res
    return res
