"""Build check, no GPU: the hot kernels must compile for gfx950 without a single vector register in scratch memory.

A tile loop that spills reloads its registers from scratch with a full wait in front of each reload; such a variant
measures two times slower and is easier to catch here than on the GPU.  hipcc's -Rpass-analysis=kernel-resource-usage
prints, per kernel, the registers it took, what it spilled and the scratch bytes per lane."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOT = ("attn_stage_kernel", "local_score_kernel", "retrieve_fused_kernel", "unit_scores_rows_kernel", "unit_scores_queries_kernel",
       "call_rank_kernel", "ingest_kernel")


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    pytest.skip("no hipcc")


@pytest.mark.parametrize("source", ["attn.hip", "score.hip", "retrieve.hip", "ingest.hip"])
def test_hot_kernels_keep_their_registers(source, tmp_path):
    cmd = [_hipcc(), "--offload-arch=gfx950", "-O3", "-std=c++17", "-c", "--offload-device-only", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Rpass-analysis=kernel-resource-usage", os.path.join(ROOT, "infllm_amd", "csrc", source), "-o",
           str(tmp_path / "out.o")]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    kernels, name = {}, None
    for line in p.stderr.splitlines():
        m = re.search(r"remark: Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            kernels[name] = {}
            continue
        m = re.search(r"remark:\s+(VGPRs Spill|ScratchSize \[bytes/lane\]|VGPRs|Occupancy \[waves/SIMD\]): (\d+)", line)
        if m and name:
            kernels[name][m.group(1)] = int(m.group(2))
    hot = {k: v for k, v in kernels.items() if any(h in k for h in HOT)}
    assert hot, f"no hot kernel found in {source}: {list(kernels)[:5]}"
    for k, v in hot.items():
        print(k[:60], v)
        assert v.get("VGPRs Spill") == 0 and v.get("ScratchSize [bytes/lane]") == 0, (k, v)
    if source == "attn.hip":                   # 8 waves per workgroup, one workgroup per CU: two waves per SIMD need <= 256 registers
        assert all(v["Occupancy [waves/SIMD]"] >= 2 for k, v in hot.items()), hot
