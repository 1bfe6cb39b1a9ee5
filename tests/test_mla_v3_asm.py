"""The generated includes of the literal-AGPR kernels (csrc/ops/attn_mla.hip with gen_mla_v3.py,
csrc/ops/attn_prefill.hip with gen_prefill_v3.py) match their generators."""
import os
import shutil
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
OPS = os.path.join(ROOT, "llmd_amd", "csrc", "ops")


def test_generated_include_is_current(tmp_path):
    gen = os.path.join(OPS, "gen_mla_v3.py")
    inc = os.path.join(OPS, "mla_v3_agpr.inc")
    before = open(inc).read()
    env = dict(os.environ)
    out = tmp_path / "copy"
    out.mkdir()
    shutil.copy(gen, out / "gen_mla_v3.py")
    subprocess.run([sys.executable, str(out / "gen_mla_v3.py")], check=True, capture_output=True, env=env)
    assert (out / "mla_v3_agpr.inc").read_text() == before


def test_prefill_v3_include_is_current(tmp_path):
    gen = os.path.join(OPS, "gen_prefill_v3.py")
    inc = os.path.join(OPS, "prefill_v3_agpr.inc")
    out = tmp_path / "copy"
    out.mkdir()
    shutil.copy(gen, out / "gen_prefill_v3.py")
    subprocess.run([sys.executable, str(out / "gen_prefill_v3.py")], check=True, capture_output=True)
    assert (out / "prefill_v3_agpr.inc").read_text() == open(inc).read()
