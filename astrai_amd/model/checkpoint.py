"""int8 W8A8 checkpoints: the quantized weights and their per-channel steps stored
next to the other parameters, so that loading does no quantization pass and no
bf16 copy of the Linear weights ever has to exist.

Same directory layout and file names as the reference's ``Checkpoint``
(astrai/serialization/checkpoint.py:16-18,143-167: ``meta.json``, ``config.json``,
``model.safetensors``), which has no slot for scales or integer weights today. Every
``Linear`` weight ``<name>.weight`` is replaced in the safetensors file by

  ``<name>.weight_int8``   int8 ``[N, K]``   (``quantize_int8_per_channel`` of the bf16 weight)
  ``<name>.weight_scale``  fp32 ``[N]``      (quantization step per output channel)

and ``meta.json`` records ``{"quantization": {"scheme": "int8_w8a8_per_channel", ...}}``.
Loading builds the decoder with its Linear weights dequantized (``int8 * step`` in
bf16, for code paths that are not int8) and hands the stored integers to the int8
policy cache and to the fused path unchanged.
"""

import json
import time
from dataclasses import asdict
from pathlib import Path
from typing import Dict, Tuple

import safetensors.torch as st
import torch

from astrai_amd.model.decoder import AutoRegressiveLM, AutoRegressiveLMConfig, Linear, fuse_int8_weights

_META_FILE = "meta.json"
_CONFIG_FILE = "config.json"
_WEIGHTS_FILE = "model.safetensors"
SCHEME = "int8_w8a8_per_channel"


def _linear_names(model: AutoRegressiveLM):
    return [name for name, mod in model.named_modules() if isinstance(mod, Linear)]


@torch.no_grad()
def save_int8_checkpoint(model: AutoRegressiveLM, save_dir: str) -> None:
    """Quantize every Linear weight per output channel (on the device the model is on)
    and write the checkpoint directory."""
    from astrai_amd.extension.ops.int8 import quantize_int8_per_channel

    path = Path(save_dir)
    path.mkdir(parents=True, exist_ok=True)
    linear = set(_linear_names(model))
    tensors: Dict[str, torch.Tensor] = {}
    tied = model.config.tie_word_embeddings
    for name, p in model.state_dict().items():
        owner = name.rsplit(".", 1)[0]
        if owner in linear and name.endswith(".weight"):
            if tied and owner == "lm_head":
                continue  # re-created from the embedding at load
            wq, sw = quantize_int8_per_channel(p.detach())
            tensors[name + "_int8"] = wq.cpu().contiguous()
            tensors[name + "_scale"] = sw.cpu().contiguous()
        else:
            tensors[name] = p.detach().cpu().contiguous()
    st.save_file(tensors, str(path / _WEIGHTS_FILE))
    meta = {
        "timestamp": time.strftime("%Y-%m-%dT%H:%M:%S"),
        "quantization": {"scheme": SCHEME, "weight_dtype": "int8", "scale_dtype": "float32",
                         "granularity": "per output channel, symmetric, step = amax / 127",
                         "activations": "int8 per token, quantized at run time"},
    }
    (path / _META_FILE).write_text(json.dumps(meta, indent=2))
    (path / _CONFIG_FILE).write_text(json.dumps(asdict(model.config), indent=2))


@torch.no_grad()
def load_int8_checkpoint(save_dir: str, device="cuda", fuse: bool = True) -> AutoRegressiveLM:
    """Build the decoder from ``save_dir`` on ``device``; the stored integers go to the int8
    policy cache (``w8a8.int8_state()``) and, with ``fuse``, to the fused int8 path."""
    from astrai_amd.extension import w8a8

    path = Path(save_dir)
    meta = json.loads((path / _META_FILE).read_text())
    if meta.get("quantization", {}).get("scheme") != SCHEME:
        raise ValueError(f"{save_dir} is not an {SCHEME} checkpoint")
    cfg = AutoRegressiveLMConfig(**json.loads((path / _CONFIG_FILE).read_text()))
    tensors = st.load_file(str(path / _WEIGHTS_FILE))  # safetensors: data only, nothing executed
    with torch.device(device):
        model = AutoRegressiveLM(cfg).to(torch.bfloat16).eval()
    quantized: Dict[str, Tuple[torch.Tensor, torch.Tensor]] = {}
    plain = {}
    for name, t in tensors.items():
        if name.endswith(".weight_int8"):
            base = name[: -len("_int8")]
            wq = t.to(device)
            sw = tensors[base + "_scale"].to(device)
            quantized[base] = (wq, sw)
            plain[base] = (wq.float() * sw.reshape(-1, 1)).to(torch.bfloat16)
        elif not name.endswith(".weight_scale"):
            plain[name] = t.to(device)
    missing, unexpected = model.load_state_dict(plain, strict=False)
    missing = [m for m in missing if not (cfg.tie_word_embeddings and m == "lm_head.weight")]
    if missing or unexpected:
        raise ValueError(f"checkpoint does not match the model: missing {missing}, unexpected {unexpected}")
    params = dict(model.named_parameters())
    state = w8a8.int8_state()
    for base, (wq, sw) in quantized.items():
        state.put_weight(params[base], wq, sw)
    if fuse:
        fuse_int8_weights(model)  # concatenates what the cache holds: the stored integers
    return model


# ---------------------------------------------------------------------------
# fp8 delayed scaling: the amax histories and steps of every Linear weight, so that a
# resumed run quantizes its next step with the steps the interrupted run had reached
# (the reference keeps them in process memory only, keyed by the weight's address:
# astrai/extension/fp8.py:111-213; its Checkpoint has no slot for them).
# ---------------------------------------------------------------------------

_FP8_FILE = "fp8_scaling.safetensors"
_RINGS = ("w", "x", "g")


@torch.no_grad()
def save_fp8_scaling(model: torch.nn.Module, save_dir: str) -> int:
    """Write ``fp8_scaling.safetensors`` into ``save_dir`` and record the recipe in
    ``meta.json`` (created, or extended if it exists). Per parameter ``<name>`` that has
    scaling state: ``<name>.fp8_{w,x,g}_hist`` fp32 ``[history_len]``, ``<name>.fp8_{w,x,g}_scale``
    fp32 ``[1]``, ``<name>.fp8_cursor`` int64 ``[3]`` (next slot of each ring) and
    ``<name>.fp8_seeded`` int64 ``[3]``. Returns the number of parameters written."""
    from astrai_amd.extension.fp8 import fp8_state

    state = fp8_state()
    path = Path(save_dir)
    path.mkdir(parents=True, exist_ok=True)
    tensors: Dict[str, torch.Tensor] = {}
    count = 0
    for name, p in model.named_parameters():
        meta = state.peek_weight_meta(p)
        if meta is None:
            continue
        count += 1
        for r in _RINGS:
            tensors[f"{name}.fp8_{r}_hist"] = getattr(meta, f"{r}_hist").detach().float().cpu().contiguous()
            tensors[f"{name}.fp8_{r}_scale"] = getattr(meta, f"{r}_scale").detach().float().cpu().contiguous()
        tensors[f"{name}.fp8_cursor"] = torch.tensor([getattr(meta, f"{r}_idx") for r in _RINGS], dtype=torch.int64)
        tensors[f"{name}.fp8_seeded"] = torch.tensor([int(getattr(meta, f"{r}_init")) for r in _RINGS], dtype=torch.int64)
    st.save_file(tensors, str(path / _FP8_FILE))
    meta_path = path / _META_FILE
    meta = json.loads(meta_path.read_text()) if meta_path.exists() else {}
    meta["fp8_scaling"] = {"recipe": type(state.recipe).__name__, "history_len": state.recipe.history_len,
                           "margin": state.recipe.margin, "fp8_format": state.fp8_format.value,
                           "parameters": count}
    meta_path.write_text(json.dumps(meta, indent=2))
    return count


@torch.no_grad()
def load_fp8_scaling(model: torch.nn.Module, save_dir: str) -> int:
    """Restore what :func:`save_fp8_scaling` wrote into the process's fp8 state, for the
    parameters of ``model`` (on whatever device they live), under the recipe that is active
    now. A history of another length is refused: its steps would not be the saved run's.
    Returns the number of parameters restored."""
    from astrai_amd.extension.fp8 import fp8_state

    state = fp8_state()
    path = Path(save_dir)
    tensors = st.load_file(str(path / _FP8_FILE))  # safetensors: data only, nothing executed
    count = 0
    for name, p in model.named_parameters():
        if f"{name}.fp8_cursor" not in tensors:
            continue
        hist_len = tensors[f"{name}.fp8_w_hist"].numel()
        if hist_len != state.recipe.history_len:
            raise ValueError(f"{name}: saved amax history has {hist_len} slots, the active recipe "
                             f"{state.recipe.history_len}")
        meta = state.get_weight_meta(p)
        cursor = tensors[f"{name}.fp8_cursor"].tolist()
        seeded = tensors[f"{name}.fp8_seeded"].tolist()
        for i, r in enumerate(_RINGS):
            getattr(meta, f"{r}_hist").copy_(tensors[f"{name}.fp8_{r}_hist"])
            getattr(meta, f"{r}_scale").copy_(tensors[f"{name}.fp8_{r}_scale"])
            setattr(meta, f"{r}_idx", int(cursor[i]) % hist_len)
            setattr(meta, f"{r}_init", bool(seeded[i]))
        meta.w_cached = None
        count += 1
    return count

