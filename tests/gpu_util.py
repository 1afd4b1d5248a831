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

# RMS gates (the verifier's metric is sqrt(sum d^2) / (max |value| * sqrt(N)),
# conv-validation-wrappers.cpp:197-215).  f32 and f16 results: the reference's
# defaults, 3e-5 and 1e-3 (rocmlir-gen.cpp:2850-2855).  For every other type the
# reference's default is also 3e-5, which a narrower type cannot meet on
# real-valued data (its tests raise the gate per case with -RMS_threshold,
# 0.001 to 0.015 under mlir/test), so the gate here is the type's own
# resolution.  The oracle is rounded through the output type before the
# comparison, so a result that differs from it does so by one unit in the last
# place: between 2^-(b+1) and 2^-b of its magnitude for b stored mantissa bits.
# Even with EVERY element one ulp off the metric stays below 2^-b (rms <= max);
# the gates are half of that, 2^-8 (bf16), 2^-4 (fp8 e4m3) and 2^-3 (bf8 e5m2).
# These types are additionally covered bit for bit by the integer-valued tests.
RMS_THRESHOLD = {"f32": 3e-5, "f16": 1e-3, "bf16": 2.0 ** -8, "fp8": 2.0 ** -4, "bf8": 2.0 ** -3}


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
