"""Writes tests/golden/sdxl_lora_keys.json from the reference's LoRA metadata fixtures.

Source data (JSON, read as text; nothing of the reference is executed):
  /root/reference/lora_info_shm/TheLastBen_Papercut_SDXL_key_match_unet.json   unet key -> lora down/up keys
  /root/reference/lora_info_shm/TheLastBen_Papercut_SDXL.json                   lora key -> {shape, nbytes}
  /root/reference/lora_info_shm/TheLastBen_Papercut_SDXL_alphas.json            alpha per module
Output: {"<unet weight key>": {"down_key": ..., "up_key": ..., "down": [r, in], "up": [out, r], "alpha": a}}
Run in the build container only (the reference tree does not exist on the GPU box).
"""
import json
from pathlib import Path

REF = Path("/root/reference/lora_info_shm")
OUT = Path(__file__).resolve().parent / "sdxl_lora_keys.json"


def main():
    match = json.loads((REF / "TheLastBen_Papercut_SDXL_key_match_unet.json").read_text())
    info = json.loads((REF / "TheLastBen_Papercut_SDXL.json").read_text())
    alphas = json.loads((REF / "TheLastBen_Papercut_SDXL_alphas.json").read_text())
    out = {}
    for unet_key, m in match.items():
        dk, uk = m["lora_down_key"], m["lora_up_key"]
        # alpha is stored under "<down key>.alpha" (attention processors) or "unet.<module>.alpha" (the rest)
        mod = unet_key[: -len(".weight")]
        alpha = alphas.get(dk + ".alpha", alphas.get("unet." + mod + ".alpha"))
        out[unet_key] = {"down_key": dk, "up_key": uk, "down": info[dk]["shape"], "up": info[uk]["shape"], "alpha": alpha}
    OUT.write_text(json.dumps(out, separators=(",", ":"), sort_keys=True))
    print(len(out), "keys ->", OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
