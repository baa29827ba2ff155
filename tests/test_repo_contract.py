"""Checks that hold without a GPU: the product never reaches into the oracle, and bench.py refuses more than one GPU."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_product_package_does_not_import_the_oracle():
  pkg = os.path.join(ROOT, "flashtensor_amd")
  offenders = []
  for dirpath, _, files in os.walk(pkg):
    for f in files:
      if f.endswith((".py", ".hip", ".h", ".hpp")):
        text = open(os.path.join(dirpath, f), encoding="utf-8", errors="replace").read()
        if re.search(r"^\s*(import|from)\s+oracle\b", text, re.M) or "oracle/" in text:
          offenders.append(os.path.relpath(os.path.join(dirpath, f), ROOT))
  assert offenders == []


def test_bench_refuses_more_than_one_gpu():
  for extra_env, argv in (({}, ["--gpus", "2"]), ({"WORLD_SIZE": "2"}, [])):
    env = dict(os.environ, **extra_env)
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + argv, capture_output=True, text=True, env=env, timeout=120)
    assert res.returncode != 0
    assert "ONE GPU" in res.stderr and res.stdout.strip() == ""


def test_header_and_binding_agree_on_the_version():
  header = open(os.path.join(ROOT, "include", "ft_abi.h")).read()
  version = int(re.search(r"#define FT_ABI_VERSION (\d+)", header).group(1))
  sys.path.insert(0, ROOT)
  from flashtensor_amd import _lib
  assert _lib.ABI_VERSION == version
