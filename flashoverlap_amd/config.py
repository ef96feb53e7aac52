"""Two-stage per-shape JSON configs, same schema and file naming as the reference.

Stage 1 (tune/gen_config.py:69-86, tune/profile_config.py:57-72):
    {"BM": [..], "BN": [..], "dur": [.. ms], "Algo": [..]}   top GEMM tile configs
Stage 2 (tune/search.py:34-51) overwrites the same keys with scalars and adds
    "hint" (tile ids in completion order), "cSeg" (tiles per group), "rLDN": 1.
File name: configs/m{M}n{N}k{K}_{gpu}.json with gpu = device_name[7:11].lower()
(tune/search.py:21-24).
"""
import json
import os

DEFAULT_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "configs")


def gpu_tag(device_name=None):
    """The reference slices characters 7..10 of the device name ("NVIDIA A800..." -> "a800");
    "AMD Instinct MI355X" gives "tinc".  Blanks are trimmed (a name like "AMD Radeon Graphics"
    would otherwise put a space into the file name).  FLASHOVERLAP_GPU_TAG overrides."""
    tag = os.environ.get("FLASHOVERLAP_GPU_TAG")
    if tag:
        return tag
    if device_name is None:
        import torch
        device_name = torch.cuda.get_device_properties(torch.cuda.current_device()).name
    return device_name[7:11].lower().strip().replace(" ", "_")


def config_path(M, N, K, gpu=None, directory=None):
    return os.path.join(directory or DEFAULT_DIR, f"m{M}n{N}k{K}_{gpu or gpu_tag()}.json")


def save_gemm_candidates(M, N, K, BM, BN, dur, Algo, gpu=None, directory=None):
    path = config_path(M, N, K, gpu, directory)
    os.makedirs(os.path.dirname(path), exist_ok=True)
    data = {"BM": list(BM), "BN": list(BN), "dur": list(dur), "Algo": list(Algo)}
    with open(path, "w", encoding="utf-8") as f:
        json.dump(data, f, indent=4)
    return path


def load_gemm_candidates(M, N, K, gpu=None, directory=None):
    path = config_path(M, N, K, gpu, directory)
    if not os.path.exists(path):
        raise FileNotFoundError(f"{path}: run the GEMM config stage first")
    with open(path, "r", encoding="utf-8") as f:
        data = json.load(f)
    return data["BM"], data["BN"], data["dur"], data["Algo"]


def save_solution(M, N, K, BM, BN, gemm_dur, Algo, hint, cSeg, gpu=None, directory=None):
    path = config_path(M, N, K, gpu, directory)
    data = {}
    if os.path.exists(path):
        with open(path, "r", encoding="utf-8") as f:
            data = json.load(f)
    else:
        os.makedirs(os.path.dirname(path), exist_ok=True)
    data.update({"hint": [int(h) for h in hint], "cSeg": [int(c) for c in cSeg], "rLDN": 1,
                 "BM": int(BM), "BN": int(BN), "dur": float(gemm_dur), "Algo": int(Algo)})
    with open(path, "w", encoding="utf-8") as f:
        json.dump(data, f, indent=4)
    return path


def load_solution(M, N, K, gpu=None, directory=None):
    with open(config_path(M, N, K, gpu, directory), "r", encoding="utf-8") as f:
        data = json.load(f)
    for key in ("hint", "cSeg", "BM", "BN", "Algo"):
        if key not in data or isinstance(data.get("BM"), list):
            raise ValueError("config holds GEMM candidates only: run the wave-group search")
    return data
