"""Fold the parameters of split BitLinear layers back into plain Linear weights.

A split layer stores `<name>.ulinear.weight` [out, r], `<name>.s` [r], `<name>.vlinear.weight` [r, in]
and, when a residual is kept, `<name>.warmup_linear.{weight,bias}`.  The plain layer it stands for has

    weight = ulinear.weight @ diag(s) @ vlinear.weight (+ warmup_linear.weight),   bias = warmup_linear.bias

which is what the reference's converter writes (tools/convert_bitlinear_to_standard.py:80-172), so a
checkpoint trained with the patched model can be loaded into the unpatched architecture again.

    python -m metis_hip.tools.merge_state_dict in.safetensors out.safetensors [--dtype bfloat16]
"""
from __future__ import annotations

import argparse
import re
from collections import OrderedDict

import torch

_PART = re.compile(r"(.+)\.(ulinear|vlinear|warmup_linear)\.(weight|bias)$")
_DTYPES = {"keep": None, "float32": torch.float32, "fp32": torch.float32, "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
           "float16": torch.float16, "fp16": torch.float16}


def _cast(t: torch.Tensor, dtype):
    return t if dtype is None or not t.is_floating_point() else t.to(dtype)


def merge_bitlinear_state_dict(state_dict, target_dtype: torch.dtype | None = None, verbose: bool = False):
    """Returns a new ordered dict with every split layer merged; all other entries pass through
    (cast to target_dtype when given).  The product is formed in float32 and stored in the residual's
    dtype (the factor's dtype when there is no residual)."""
    prefixes = sorted({m.group(1) for m in map(_PART.match, state_dict) if m})
    out: OrderedDict[str, torch.Tensor] = OrderedDict()
    consumed = set()
    for p in prefixes:
        u, v, s = (state_dict.get(f"{p}.{k}") for k in ("ulinear.weight", "vlinear.weight", "s"))
        res_w, res_b, u_b = (state_dict.get(f"{p}.{k}") for k in ("warmup_linear.weight", "warmup_linear.bias", "ulinear.bias"))
        consumed.update(k for k in (f"{p}.ulinear.weight", f"{p}.ulinear.bias", f"{p}.vlinear.weight", f"{p}.vlinear.bias",
                                    f"{p}.s", f"{p}.warmup_linear.weight", f"{p}.warmup_linear.bias") if k in state_dict)
        if u is not None and v is not None and s is not None:
            w = (u.float() * s.float()) @ v.float()
            if res_w is not None:
                w = (w + res_w.float()).to(res_w.dtype)
            else:
                w = w.to(u.dtype)
            out[f"{p}.weight"] = _cast(w, target_dtype)
            bias = res_b if res_b is not None else u_b
            if bias is not None:
                out[f"{p}.bias"] = _cast(bias, target_dtype)
            if verbose:
                print(f"merged {p}: U diag(s) V{' + residual' if res_w is not None else ''} -> {tuple(w.shape)}")
        elif res_w is not None:                                  # patched but never split
            out[f"{p}.weight"] = _cast(res_w, target_dtype)
            if res_b is not None:
                out[f"{p}.bias"] = _cast(res_b, target_dtype)
        else:
            raise KeyError(f"{p}: neither a complete factorisation (ulinear.weight, s, vlinear.weight) nor warmup_linear.weight")
    for k, t in state_dict.items():
        if k not in consumed:
            out[k] = _cast(t, target_dtype)
    return out


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("src", help="safetensors file with BitLinear parameters")
    ap.add_argument("dst", help="safetensors file to write")
    ap.add_argument("--dtype", default="keep", choices=sorted(_DTYPES))
    ap.add_argument("-v", "--verbose", action="store_true")
    args = ap.parse_args(argv)
    from safetensors.torch import load_file, save_file
    merged = merge_bitlinear_state_dict(load_file(args.src), _DTYPES[args.dtype], args.verbose)
    save_file({k: t.contiguous() for k, t in merged.items()}, args.dst)
    print(f"{args.src}: wrote {len(merged)} tensors to {args.dst}")


if __name__ == "__main__":
    main()
