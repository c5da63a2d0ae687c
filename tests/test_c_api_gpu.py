"""The engine's C ABI (capi/tli_engine.h) as a C program uses it: tests/c_api_client.c is compiled
against the header and libtli_engine.so, serves three requests of a tiny model and prints their
tokens, which are the plain implementation's greedy ones in float32."""
import os
import shutil
import subprocess

import pytest

import plain_qwen3
from helpers import random_prompt

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_a_c_program_generates_through_the_engine(model_folders, tmp_path):
    from tiny_llm_infer_amd.kernels import build
    lib = build.find_engine_api() or build.build_engine_api()
    cc = shutil.which("gcc") or shutil.which("cc")
    assert cc, "no C compiler"
    capi = os.path.dirname(lib)
    exe = str(tmp_path / "client")
    proc = subprocess.run([cc, "-O1", os.path.join(ROOT, "tests", "c_api_client.c"), f"-I{capi}", f"-L{capi}", "-ltli_engine",
                           f"-Wl,-rpath,{capi}", "-o", exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout
    folder = model_folders["A"]
    cfg, w = plain_qwen3.read_model(folder)
    prompts = [random_prompt(256, n, 40 + n) for n in (5, 17, 33)]
    want = [plain_qwen3.greedy(cfg, w, p, 10) for p in prompts]
    run = subprocess.run([exe, folder, "float32", "10"] + [",".join(map(str, p)) for p in prompts],
                         stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    lines = run.stdout.strip().split("\n")
    assert [list(map(int, line.split())) for line in lines[:3]] == want
    assert lines[3] == "generated 30"
    assert "refused as expected" in run.stderr and "vocabulary" in run.stderr
