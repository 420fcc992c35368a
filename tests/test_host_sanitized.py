"""The host layer (host/*.cpp and the class headers it instantiates) under AddressSanitizer and
UndefinedBehaviorSanitizer, without a GPU: the device entry points are replaced by host stand-ins
and tests/cpp/host_replay.cpp replays what the encoder-stack tests do through the C ABI (pattern
generation, model assembly, forwards, changed lengths and masks, the archive loader, error paths).
Any access outside a buffer on those paths, or undefined arithmetic, fails the run."""
import re
import subprocess
from pathlib import Path

import numpy as np
import pytest

from oracle import formats as F

ROOT = Path(__file__).resolve().parent.parent
PKG = ROOT / "scpaper-2021_amd"
CPP = ROOT / "tests" / "cpp"
CLANG = Path("/opt/rocm/lib/llvm/bin/clang++")


def abi_functions() -> list[str]:
    text = "\n".join(h.read_text() for h in sorted((ROOT / "include").glob("*.h")))  # et_abi.h, et_tuning.h
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"^\s*(?:const\s+char\s*\*|int|void)\s*(et_\w+)\s*\(", text, flags=re.M)))


def defined_in(paths) -> set[str]:
    names = set()
    for p in paths:
        names |= set(re.findall(r"^\s*(?:const\s+char\s*\*|int|void)\s*(et_\w+)\s*\(", p.read_text(), flags=re.M))
    return names


@pytest.fixture(scope="module")
def replay_binary(tmp_path_factory):
    if not CLANG.exists():
        pytest.skip("the ROCm clang++ is not installed")
    build = tmp_path_factory.mktemp("host_sanitized")
    host_sources = sorted((PKG / "host").glob("*.cpp"))
    have = defined_in(host_sources + [CPP / "device_stubs_base.cpp"])
    generated = build / "device_stubs_generated.cpp"
    generated.write_text('extern "C" {\n' + "".join(f"int {n}() {{ return 0; }}\n" for n in abi_functions()
                                                    if n not in have) + "}\n")
    exe = build / "host_replay"
    cmd = [str(CLANG), "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
           "-fno-omit-frame-pointer", "-I", str(ROOT / "include"), str(CPP / "host_replay.cpp"),
           str(CPP / "device_stubs_base.cpp"), str(generated), *map(str, host_sources), "-lz", "-o", str(exe)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-4000:]
    return exe


def write_small_model(directory: Path):
    """Archives of a 2-layer H128 nh2 FF256 model in the exporter's layout (numpy's own writer)."""
    rng = np.random.default_rng(3)
    names = []
    for layer in range(2):
        pre = f"transformer_encoder.layers.{layer}."
        for nm, (o, i) in (("self_attn.in_proj_", (384, 128)), ("self_attn.out_proj.", (128, 128)),
                           ("linear1.", (256, 128)), ("linear2.", (128, 256))):
            W = rng.standard_normal((o, i)).astype(np.float32)
            mask = rng.random((o // 16, i // 16)) < 0.5
            W = (W.reshape(o // 16, 16, i // 16, 16) * mask[:, None, :, None]).reshape(o, i)
            F.save_weight_npz(str(directory / (pre + nm)), W, rng.standard_normal(o).astype(np.float32))
            names.append(pre + nm + ".npz")
        for nm in ("norm1.", "norm2."):
            F.save_weight_npz(str(directory / (pre + nm)), np.ones(128, np.float32), np.zeros(128, np.float32))
            names.append(pre + nm + ".npz")
    (directory / "weights.txt").write_text("\n".join(names) + "\n")


def test_host_layer_is_clean_under_sanitizers(replay_binary, tmp_path):
    write_small_model(tmp_path)
    env = {"ASAN_OPTIONS": "detect_leaks=1:abort_on_error=0", "UBSAN_OPTIONS": "print_stacktrace=1",
           "PATH": "/usr/bin:/bin"}
    res = subprocess.run([str(replay_binary), str(tmp_path)], capture_output=True, text=True, env=env, timeout=600)
    assert res.returncode == 0 and "host_replay ok" in res.stdout, (res.stdout + res.stderr)[-6000:]
    assert "Sanitizer" not in res.stderr and "runtime error" not in res.stderr, res.stderr[-6000:]
