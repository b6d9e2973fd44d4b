"""Seeded sweep over layer shapes, batch sizes and activity masks against the
CPU oracle, through the C-ABI: expert counts that are no power of two, hidden
sizes that leave a narrow last column tile or are no multiple of 64 (padded
inside the library), batch sizes on both sides of every size at which the
library changes its plan, handles larger than the batch.

Bars as in test_gpu_parity.py: ids, offsets and permutations bit-exact; outputs
within max-abs 2e-2 and rel-L2 1e-3 of the oracle on the same bf16 inputs."""
import numpy as np
import pytest

from gpt_oss_amd import abi, synth
from oracle import binding as ob

pytestmark = pytest.mark.gpu

W = ("w_router", "b_router", "w_mlp1", "b_mlp1", "w_mlp2", "b_mlp2")
EXPERTS = [4, 5, 8, 13, 16, 32, 33, 64, 100, 128, 200, 256]
HIDDEN = [32, 64, 96, 128, 192, 320]
INTER = [32, 64, 96, 128, 256]
TOKENS = [1, 2, 15, 16, 17, 63, 64, 65, 100, 128, 129, 255, 256, 257, 300, 511, 513, 1000, 1500, 2500]


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5])
def test_random_shapes(seed):
    rng = np.random.default_rng(seed)
    for _ in range(25):
        E, H, IM, T = (int(rng.choice(v)) for v in (EXPERTS, HIDDEN, INTER, TOKENS))
        sh = synth.LayerShape("r", T, H, IM, E, zipf=float(rng.choice([0.0, 0.0, 1.2])))
        L = synth.make_layer(sh, seed=int(rng.integers(1 << 30)))
        L = {k: (synth.round_bf16(v) if v.dtype == np.float32 else v) for k, v in L.items()}
        x = L["x"]
        pos = None
        if rng.random() < 0.5:
            pos = np.zeros(T, np.int32)
            pos[rng.random(T) < rng.choice([0.05, 0.5, 0.95])] = -1
        case = f"E={E} H={H} IM={IM} T={T} masked={pos is not None}"
        m = abi.Moe(H, IM, E, max_tokens=int(rng.choice([T, T + 7, 4096 + T])), swiglu_limit=sh.limit)
        m.upload_layer(0, *[L[k] for k in W])
        R = abi.run_layer(m, 0, x, pos)
        _, ti, _ = ob.router(x, pos, L["w_router"], L["b_router"], 4)
        off, perm, _ = ob.dispatch(ti, pos, E)
        assert np.array_equal(R["topk_i"], ti), case
        assert np.array_equal(R["offsets"], off) and np.array_equal(R["perm"][:off[-1]], perm), case
        assert np.all(R["perm"][off[-1]:] == -1), case
        rows = np.sort(rng.choice(T, min(T, 32), replace=False))
        want = ob.moe_layer(np.ascontiguousarray(x[rows]), None if pos is None else np.ascontiguousarray(pos[rows]),
                            *[L[k] for k in W], 4, sh.limit, mode=ob.ROUND_ACT_BF16 | ob.PAR_TOKENS)
        got = R["out"][rows]
        assert np.abs(got - want).max() <= 2e-2, case
        assert np.linalg.norm(got - want) <= 1e-3 * max(np.linalg.norm(want), 1e-30), case
        if pos is not None:
            assert np.all(R["out"][pos < 0] == 0), case
        m.close()
