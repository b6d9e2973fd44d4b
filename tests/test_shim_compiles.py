"""The C++17 host shim compiles against the reference's own types (Transformer,
DeviceContext, Config) and links against the C-ABI library.  Needs the reference
checkout, so it runs in the build container only.  No GPU."""
import os
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"

TU = r'''
#define TESTING
#include "%(ref)s/run.cpp"
#include "expert_mi355.hpp"
// uses every shim entry point with the reference's argument lists
void shim_smoke(Transformer *t) {
  DeviceContext ctx; ctx.device_id = 0;
  mi355_moe_init(ctx, 0, t, MAX_BATCH_SIZE);
  Config *p = &t->config;
  mi355_moe_forward(ctx, p->swiglu_limit, p->hidden_dim, p->intermediate_dim, p->n_experts,
                    p->n_layers, p->experts_per_token, 1, 0);
  mi355_moe_forward_fused(ctx, 1, 0);
  mi355_moe_cleanup(ctx);
}
'''


@pytest.mark.skipif(not os.path.exists(os.path.join(REF, "run.cpp")), reason="reference checkout not present")
def test_shim_compiles_against_reference_types():
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "tu.cpp")
        open(src, "w").write(TU % {"ref": REF})
        cmd = ["/opt/rocm/bin/hipcc", "--std=c++17", "--offload-arch=gfx950", "-fopenmp", "-include",
               "thread", "-w", "-I", REF, "-I", os.path.join(ROOT, "include"), "-I",
               os.path.join(ROOT, "gpt_oss_amd", "shim"), "-c", src, "-o", os.path.join(d, "tu.o")]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-3000:]
