"""The host half of the library (plan.cpp) under AddressSanitizer + UBSan: valid tables of the
fixture programs are accepted, thousands of randomly corrupted copies are refused without a crash."""
import os
import subprocess

import numpy as np
import pytest

import golden_util
import ir_samples
from msccl.executor import parse_algo_xml

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "msccl-tools_amd", "csrc")


@pytest.fixture(scope="module")
def driver(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("fuzz") / "host_plan_fuzz")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-I", os.path.join(ROOT, "include"),
           "-I", CSRC, os.path.join(ROOT, "tests", "host_plan_fuzz.cpp"), os.path.join(CSRC, "plan.cpp"), "-o", exe]
    subprocess.run(cmd, check=True)
    return exe


def dump(tables, path):
    with open(path, "wb") as f:
        np.array([tables.ngpus, tables.ntbs, tables.nops], np.int32).tofile(f)
        np.ascontiguousarray(tables.rank_chunks, np.int32).tofile(f)
        np.ascontiguousarray(tables.tbs, np.int32).tofile(f)
        np.ascontiguousarray(tables.ops, np.int32).tofile(f)


@pytest.mark.parametrize("name,mutations", [("fusion_chain", 4000), ("allpairs_sample", 3000), ("c3_alltoall_two_step_2x8", 1500),
                                            ("allreduce_a100_ncv4_8r", 3000), ("alltonext_forward_2x8", 1500),
                                            ("c4_hierarchical_allreduce_8x4_2inst_auto", 60)])
def test_plan_builder_survives_corrupted_tables(driver, tmp_path, name, mutations):
    xml = {"fusion_chain": ir_samples.FUSION_CHAIN_XML, "allpairs_sample": ir_samples.allpairs_allreduce_xml(4)}.get(name) or golden_util.load(name)
    path = str(tmp_path / "tables.bin")
    dump(parse_algo_xml(xml), path)
    # (verify_asan_link_order=0: the sanitizer runtime tolerates libraries preloaded ahead of it)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:verify_asan_link_order=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([driver, path, str(mutations)], capture_output=True, text=True, env=env, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-4000:]
    assert f"ok: {mutations} mutated tables handled" in r.stdout
