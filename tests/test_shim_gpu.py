"""Runs tests/cpp/shim_test: the C++ shim (namespace ms::q over the C ABI) with known answers and the abort contract."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "shim_test")


def test_shim_header_declares_the_reference_operator_names():
    text = open(os.path.join(ROOT, "include", "macseek_amd", "quant.hpp")).read()
    for name in ("matvec_supported", "matvec_cfg", "encode_matvec", "encode_matvec_n", "moe_decode_scratch_bytes",
                 "encode_moe_decode", "encode_moe_decode_table", "encode_moe_decode_table_part", "moe_prefill_scratch_bytes",
                 "encode_moe_prefill", "struct MvCfg", "struct ExpertSlot", "struct MoeDecodeArgs", "struct MoePrefillArgs",
                 "enum class MoePart", "kExpertDim", "kExpertInter", "kMaxRouted"):
        assert name in text, name


@pytest.mark.gpu
def test_cpp_shim_program(dev):
    assert os.path.exists(EXE), "tests/cpp/shim_test is not built (python -m macseek_amd.build)"
    env = dict(os.environ, LD_LIBRARY_PATH=os.path.join(ROOT, "macseek_amd") + ":" + os.environ.get("LD_LIBRARY_PATH", ""))
    r = subprocess.run([EXE], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120, env=env)
    print(r.stdout)
    assert r.returncode == 0 and "all OK" in r.stdout
