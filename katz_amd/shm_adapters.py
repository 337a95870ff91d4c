"""Katz's shared-memory adapter hand-off: the layout a CPU loader process writes and the UNet process reads.

Layout (load_lora_shm_multi.py:40-61, :107-121; pipeline_controlnet_sd_xl_katz.py:253-280), kept as is:
  * one POSIX shared-memory segment per adapter tensor, named "<lora key>_<loader id>", holding a C-contiguous
    float16 array of the shape listed in the adapter's metadata JSON ({key: {"shape": [...], "nbytes": n}});
  * one segment "start_loading_flag": int8[n_loaders]; per loader 0 = idle, 1 / 2 = "load adapter 1 / 2" (set by the
    UNet process), 10 = tensors are in place (set by the loader), 100 = shut down;
  * sidecars "<repo>_alphas.json" ({"<module>.alpha": a}) and "<repo>_key_match_unet.json"
    ({"<unet weight key>": {"lora_down_key": k, "lora_up_key": k}}).

`ShmAdapterSegments` opens (or, for a loader / a test, creates) the segments and hands the tensors out as torch
views without copying.  Two consumers: `UNet2DConditionModel.load_lora_into_unet(reader.state_dict(), alphas)`
packs them for the LoRA kernels (no merge at all), and `patch_on_lora` below is Katz's merge path
(pipeline_controlnet_sd_xl_katz.py:1730-1747) as in-place GEMMs on the GPU.
"""
from __future__ import annotations

import json
from multiprocessing import shared_memory
from typing import Dict, Mapping, Optional

import numpy as np
import torch

from . import ops

FLAG_NAME = "start_loading_flag"
IDLE, LOADED, SHUTDOWN = 0, 10, 100


def read_info(path_or_dict) -> Dict[str, dict]:
    if isinstance(path_or_dict, Mapping):
        return dict(path_or_dict)
    with open(path_or_dict, "r") as fr:
        return json.load(fr)


class ShmAdapterSegments:
    """The segments of one loader.  create=True plays the loader's side (load_lora_shm_multi.py:47-61);
    create=False the pipeline's (pipeline_controlnet_sd_xl_katz.py:253-280).  name_prefix isolates tests from
    each other; Katz uses none."""

    def __init__(self, info, loader_id: int = 0, n_loaders: int = 2, create: bool = False, name_prefix: str = ""):
        self.info = read_info(info)
        self.loader_id, self.n_loaders, self.created, self.prefix = loader_id, n_loaders, create, name_prefix
        self._shm: Dict[str, shared_memory.SharedMemory] = {}
        self.arrays: Dict[str, np.ndarray] = {}
        flag_name = name_prefix + FLAG_NAME
        try:
            self._flag_shm = shared_memory.SharedMemory(name=flag_name, create=create and loader_id == 0, size=n_loaders if create and loader_id == 0 else 0)
        except FileNotFoundError as e:
            raise FileNotFoundError(f"shared-memory segment {flag_name!r} does not exist: no loader process has created it") from e
        self.flags = np.ndarray((n_loaders,), dtype=np.int8, buffer=self._flag_shm.buf)
        if create:
            self.flags[loader_id] = IDLE
        for key, meta in self.info.items():
            shape = tuple(meta["shape"])
            nbytes = int(np.prod(shape)) * 2
            if int(meta.get("nbytes", nbytes)) != nbytes:
                raise ValueError(f"{key}: nbytes {meta['nbytes']} does not match float16 {shape}")
            seg = shared_memory.SharedMemory(name=f"{name_prefix}{key}_{loader_id}", create=create, size=nbytes if create else 0)
            self._shm[key] = seg
            self.arrays[key] = np.ndarray(shape, dtype=np.float16, buffer=seg.buf)
            if create:
                self.arrays[key].fill(0)

    # ---- loader side ------------------------------------------------------------------------------------------
    def publish(self, state_dict: Mapping[str, torch.Tensor]) -> None:
        """Copy an adapter's tensors into the segments and raise the flag to 10 (load_lora_shm_multi.py:113-118)."""
        for key, arr in self.arrays.items():
            arr[:] = state_dict[key].detach().to(torch.float16).cpu().numpy()[:]
        self.flags[self.loader_id] = LOADED

    # ---- pipeline side -----------------------------------------------------------------------------------------
    def request(self, which: int = 1) -> None:
        self.flags[self.loader_id] = which

    def loaded(self) -> bool:
        return int(self.flags[self.loader_id]) == LOADED

    def state_dict(self) -> Dict[str, torch.Tensor]:
        """Zero-copy float16 CPU tensors over the segments (valid until close())."""
        if not self.loaded():
            raise RuntimeError(f"loader {self.loader_id} has not published its tensors (flag {int(self.flags[self.loader_id])}, need {LOADED})")
        return {k: torch.from_numpy(a) for k, a in self.arrays.items()}

    def clear(self) -> None:
        """clear_shm, pipeline_controlnet_sd_xl_katz.py:1772-1777."""
        for a in self.arrays.values():
            a.fill(0)

    def close(self) -> None:
        self.arrays.clear()
        self.flags = None
        for seg in list(self._shm.values()) + [self._flag_shm]:
            seg.close()
        if self.created:
            for seg in self._shm.values():
                seg.unlink()
            if self.loader_id == 0:
                self._flag_shm.unlink()
        self._shm.clear()


KATZ_MERGE_SCALE = 20000.0 / 64.0   # alpha / rank, hard-coded in the reference (pipeline_controlnet_sd_xl_katz.py:1737)


def patch_on_lora(unet, lora_state_dict: Mapping[str, torch.Tensor], key_match: Mapping[str, Mapping[str, str]],
                  scale: float = KATZ_MERGE_SCALE) -> int:
    """Katz's merge: for every matched UNet weight, W += (up @ down) * scale
    (pipeline_controlnet_sd_xl_katz.py:1730-1747), in place on the GPU weights.  The adapter matrices are uploaded as
    they are (float16 in Katz's shared-memory layout, or bfloat16) and ALL layers are merged by one launch of the
    batched merge kernel (kh_lora_merge_grouped_bf16): products on the matrix cores in the adapters' own dtype, fp32
    accumulation, W + scale * product rounded once (the reference rounds up @ down and the scaled product to fp16
    first, and writes the result back with load_state_dict).  Returns the number of patched weights."""
    params = dict(unet.named_parameters())
    ws, ups, downs = [], [], []
    for wkey, m in key_match.items():
        if wkey not in params:
            raise KeyError(f"{wkey} is not a parameter of the UNet")
        w = params[wkey]
        if not w.is_cuda or w.dtype != torch.bfloat16 or w.dim() != 2 or not w.is_contiguous():
            raise ValueError(f"{wkey}: patch_on_lora needs a contiguous 2-D bfloat16 GPU weight")
        down, up = lora_state_dict[m["lora_down_key"]], lora_state_dict[m["lora_up_key"]]
        n_out, n_in = w.shape
        r = down.shape[0]
        if down.shape != (r, n_in) or up.shape != (n_out, r):
            raise ValueError(f"{wkey}: adapter shapes {tuple(up.shape)} x {tuple(down.shape)} do not match {tuple(w.shape)}")
        if down.dtype not in (torch.float16, torch.bfloat16):
            down, up = down.to(torch.bfloat16), up.to(torch.bfloat16)
        ws.append(w.data)
        downs.append(down.to(w.device, non_blocking=True).contiguous())
        ups.append(up.to(w.device, non_blocking=True).contiguous())
    with torch.no_grad():
        ops.lora_merge_grouped(ws, ups, downs, scale=scale)
    for wkey in key_match:
        torch.autograd.graph.increment_version(params[wkey])   # `.data` above is a separate version counter
    return len(ws)
