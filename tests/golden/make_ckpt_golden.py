"""Writes tests/golden/ckpt_reference.json: what the REFERENCE's model-folder loader (engine/core/checkpoint.cpp,
ModelWeights::load, built from the reference's own sources by `make -C oracle ckptref` and run over the reference's CPU
backend) holds for the folders tests/folders.py writes: per target format, every projection's format, shape, the SHA-256
of its data, scale and per-expert global bytes, its scalar global, and the plain tensors' types, shapes and bytes.
Run where /root/reference is present:

    make -C oracle ref ckptref && python tests/golden/make_ckpt_golden.py

The folders' tensors are hashed too ("inputs"), so a test can tell a folder that differs from the one the fixture was made
from apart from a loader that differs from the reference.
"""

import hashlib
import json
import subprocess
import sys
import tempfile
from pathlib import Path

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
sys.path.insert(0, str(HERE.parent))
sys.path.insert(0, str(ROOT))

import folders  # noqa: E402

DUMP = ROOT / "oracle" / "_ref" / "ckptref_dump"
LAYOUTS = ("bf16", "fp8", "nvfp4")
TARGETS = {"bf16": 0, "int8": 1, "fp8": 2, "nvfp4": 3, "bf16x": 4}
SEED = 11


def sha(b):
    return hashlib.sha256(bytes(b)).hexdigest()


def run(directory, target, skip, blob, plain, skipped):
    args = [str(DUMP), str(directory), str(target), str(int(skip)), str(folders.V), str(folders.H), str(folders.E), str(folders.I),
            str(folders.L), str(blob)] + plain + (["--skipped"] + skipped if skipped else [])
    out = subprocess.run(args, check=True, capture_output=True, text=True).stdout
    data = Path(blob).read_bytes()
    case = {"projections": {}, "plain": {}, "skipped": {}}
    for line in out.splitlines():
        f = line.split()
        if f[0] == "error":
            return {"stored": case["stored"], "error": line[len("error "):]}
        if f[0] in ("stored", "format", "device_bytes"):
            case[f[0]] = int(f[1])
        elif f[0] == "projection":
            name, typ, E, N, K, stack, d0, dn, s0, sn, gbits, g0, gn, ed, es = f[1], *map(int, f[2:])
            case["projections"][name] = {"type": typ, "E": E, "N": N, "K": K, "stack": stack, "data": sha(data[d0:d0 + dn]),
                                         "data_bytes": dn, "scale": sha(data[s0:s0 + sn]) if sn else None, "scale_bytes": sn,
                                         "global_bits": gbits, "globals": sha(data[g0:g0 + gn]) if gn else None,
                                         "expert_bytes": [ed, es]}
        elif f[0] == "skipped":
            name, E, N, K, stack, ed, es, held = f[1], *map(int, f[2:])
            case["skipped"][name] = {"E": E, "N": N, "K": K, "stack": stack, "expert_bytes": [ed, es], "held": held}
        elif f[0] == "plain":
            name, dtype, rank = f[1], int(f[2]), int(f[3])
            dims = [int(v) for v in f[4:4 + rank]]
            at, n = int(f[4 + rank]), int(f[5 + rank])
            case["plain"][name] = {"dtype": dtype, "shape": dims, "bytes": sha(data[at:at + n])}
    return case


def main():
    if not DUMP.exists():
        sys.exit(f"{DUMP} is not built: make -C oracle ref ckptref (needs /root/reference)")
    golden = {"made_by": "tests/golden/make_ckpt_golden.py over oracle/_ref/ckptref_dump", "seed": SEED, "wide": True,
              "dims": {"V": folders.V, "H": folders.H, "L": folders.L, "I": folders.I, "E": folders.E}, "inputs": {}, "cases": {}}
    plain = folders.plain(wide=True)
    experts = [p for p in folders.projections(wide=True) if "local_experts." in p]
    with tempfile.TemporaryDirectory() as tmp:
        tmp = Path(tmp)
        for layout in LAYOUTS:
            tensors = folders.write(tmp / layout, layout, seed=SEED, shards=1, wide=True)
            golden["inputs"][layout] = folders.digest(tensors)
            for tname, target in TARGETS.items():
                golden["cases"][f"{layout}->{tname}"] = run(tmp / layout, target, False, tmp / "blob", plain, [])
            own = {"bf16": "int8", "fp8": "fp8", "nvfp4": "nvfp4"}[layout]
            golden["cases"][f"{layout}->{own} skip_experts"] = run(tmp / layout, TARGETS[own], True, tmp / "blob", plain, experts)
    (HERE / "ckpt_reference.json").write_text(json.dumps(golden, indent=0, sort_keys=True, separators=(",", ":")) + "\n")
    print(f"{len(golden['cases'])} cases written")


if __name__ == "__main__":
    main()
