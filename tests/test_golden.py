"""The committed golden vectors (tests/golden/exact_vectors.json, worked out with exact rational arithmetic by
tests/golden/make_exact_vectors.py from the reference's formulas, sharing no code with the oracle or the kernels)
against the CPU oracle, and -- marked gpu -- against the HIP kernels through the C ABI."""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "exact_vectors.json")) as f:
    CASES = json.load(f)["cases"]


def arrays(case):
    rows, cols = case["rows"], case["cols"]
    if case["dtype"] == "bf16":
        x = np.array(case["x_bits"], dtype=np.uint16).reshape(rows, cols)
    else:
        x = np.array(case["x_bits"], dtype=np.uint32).view(np.float32).reshape(rows, cols)
    u = None if case["u_bits"] is None else np.array(case["u_bits"], dtype=np.uint32).view(np.float32).reshape(rows, cols)
    nib = np.array(case["nibbles"], dtype=np.uint8).reshape(rows, cols)
    codes = (nib[:, 0::2] | (nib[:, 1::2] << 4)).astype(np.uint8)       # element 2i in the low nibble of byte i
    scales = np.array(case["scales"], dtype=np.uint8).reshape(rows, cols // 32)
    mask = None
    if case["mask"] is not None:
        bits = np.array(case["mask"], dtype=np.uint8).reshape(rows, cols // 8, 8)
        mask = (bits << np.arange(8, dtype=np.uint8)).sum(axis=2).astype(np.uint8)  # bit i of byte j = element 8j+i
    return x, u, codes, scales, mask


def test_the_file_is_what_the_script_writes(tmp_path):
    """The fixture is reproducible from its committed generator (pure Python, seeded)."""
    import importlib.util
    import shutil
    src = os.path.join(HERE, "golden", "make_exact_vectors.py")
    dst = tmp_path / "make_exact_vectors.py"
    shutil.copy(src, dst)
    spec = importlib.util.spec_from_file_location("make_exact_vectors", dst)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.main()
    with open(tmp_path / "exact_vectors.json") as f:
        assert json.load(f)["cases"] == CASES
    assert len(CASES) == 32


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_oracle_reproduces_the_golden_vectors(oracle, case):
    x, u, codes, scales, mask = arrays(case)
    r = oracle.quantize(x, case["hd"], signs=case["signs"], mode=case["mode"], u=u, want_mask=mask is not None)
    assert np.array_equal(r["scales"], scales)
    assert np.array_equal(r["codes"], codes)
    if mask is not None:
        assert np.array_equal(r["mask"], mask)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_kernels_reproduce_the_golden_vectors(case):
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from quartet_amd import kernels as K
    from tests.util import sign_int
    print(f"case golden {case['name']}", flush=True)
    x, u, codes, scales, mask = arrays(case)
    if case["dtype"] == "bf16":
        xt = torch.from_numpy(x.view(np.int16)).view(torch.bfloat16).cuda()
    else:
        xt = torch.from_numpy(x).cuda()
    ut = None if u is None else torch.from_numpy(u).cuda().contiguous()
    signs = 0 if case["signs"] is None else sign_int(np.array(case["signs"]))
    got = K.quantize_mxfp4(xt.contiguous(), case["hd"], signs, case["mode"], u=ut, want_mask=mask is not None)
    assert np.array_equal(got[1].cpu().numpy(), scales)
    assert np.array_equal(got[0].cpu().numpy(), codes)
    if mask is not None:
        assert np.array_equal(got[2].cpu().numpy(), mask)
