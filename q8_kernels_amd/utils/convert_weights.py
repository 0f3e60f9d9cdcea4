"""Conversion of a 16-bit LTX-Video transformer state dict to the 8-bit on-disk format of the reference
(reference: q8_kernels/utils/convert_weights.py:23-78).

Inside `transformer_blocks.*`: attention and feed-forward weight matrices become Hadamard-rotated int8 codes
(`...weight`) plus fp32 per-output-channel scales (`...scales`), biases and norm weights become fp32, and the
keys are renamed to the module tree of q8_kernels_amd.modules (`to_out.0.` -> `to_out.`, `.net.0.` -> `.act.`,
`.net.2.` -> `.proj_down.`); `scale_shift_table` and everything outside the transformer blocks is passed through.
A converted state dict loads into Q8Linear / Attention / FeedForward / LTXTransformerBlock of this package and
of the reference alike.

    python -m q8_kernels_amd.utils.convert_weights --input_path in.safetensors --output_path out.safetensors
"""
import argparse
import os
from pathlib import Path
from typing import Dict, Optional, Tuple

import torch

_PREFIX = "transformer_blocks"


def converted_key(key: str) -> Tuple[str, str]:
    """(new key, treatment) for one key of the original state dict; treatment is one of
    'quantize' (weight matrix -> int8 codes + '<...>scales'), 'fp32' (cast) and 'keep'."""
    if _PREFIX not in key:
        return key, "keep"
    if "attn" in key:
        new_key = key.replace("to_out.0.", "to_out.")
        if "norm" in key and "weight" in key:
            return new_key, "fp32"
        if "bias" in key:
            return new_key, "fp32"
        if "weight" in key:
            return new_key, "quantize"
        raise KeyError("unexpected attention key %s" % key)
    if "ff" in key:
        new_key = key.replace(".net.0.", ".act.").replace(".net.2.", ".proj_down.")
        if "bias" in key:
            return new_key, "fp32"
        if "weight" in key:
            return new_key, "quantize"
        raise KeyError("unexpected feed-forward key %s" % key)
    if "scale_shift_table" in key:
        return key, "keep"
    raise KeyError("unexpected transformer block key %s" % key)


def convert_state_dict(orig_state_dict: Dict[str, torch.Tensor], device: Optional[torch.device] = None
                       ) -> Dict[str, torch.Tensor]:
    """Returns the converted state dict; quantization runs on `device` (default: the current GPU)."""
    from ..functional.fast_hadamard import hadamard_transform
    from ..functional.quantizer import quantize
    device = torch.device("cuda") if device is None else device
    new_state_dict = {}
    for key, value in orig_state_dict.items():
        new_key, how = converted_key(key)
        if how == "quantize":
            w_quant, w_scales = quantize(hadamard_transform(value.to(device).to(torch.bfloat16)))
            new_state_dict[new_key] = w_quant
            new_state_dict[new_key.replace("weight", "scales")] = w_scales
        elif how == "fp32":
            new_state_dict[new_key] = value.float()
        else:
            new_state_dict[new_key] = value
    return new_state_dict


def load_unet(unet_path: Path) -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file
    if os.path.isdir(str(unet_path)):
        unet_path = unet_path / "unet_diffusion_pytorch_model.safetensors"
    assert unet_path.name.endswith(".safetensors"), f"{unet_path} is not a safetensors file"
    assert unet_path.exists(), f"{unet_path} does not exist"
    return load_file(str(unet_path))


def main():
    from safetensors.torch import save_file
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("--input_path", type=Path, required=True)
    parser.add_argument("--output_path", type=Path, required=True)
    args = parser.parse_args()
    new_state_dict = convert_state_dict(load_unet(args.input_path))
    save_file({k: v.contiguous().cpu() for k, v in new_state_dict.items()}, str(args.output_path))
    print(f"converted state dict saved in {args.output_path}")


if __name__ == "__main__":
    main()
