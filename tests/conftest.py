import gzip
import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (MI355X); run with -m gpu")


def load_golden(name: str):
    with gzip.open(os.path.join(GOLDEN, name), "rb") as f:
        return json.loads(f.read())


PLAN_FIELDS = ("MNWs", "q_tables", "block_tables", "num_seqs_per_CTAs", "CTA_ranks", "kv_in_CTAs",
               "num_split_per_seq", "max_split_per_seq", "max_seqs_in_CTA", "max_blocks_in_CTA")


def plan_fields(ki) -> dict:
    """KernelInfo (or the oracle's PlanResult) -> plain dict of lists."""
    return json.loads(json.dumps({k: getattr(ki, k) for k in PLAN_FIELDS}))


def run_plan_case(cls, case: dict) -> dict:
    """Runs one golden case through a scheduler class with the PrefixTree interface."""
    try:
        t = cls(case["block_size"])
        t.build_radix_tree(list(case["seq_lens"]), [list(r) for r in case["rows"]])
        plans = []
        for c in case["calls"]:
            if c["kind"] == "naive":
                ki = t.naive_schedule(c["HRatio"])
            else:
                ki = t.pack_schedule(c["MNWs"], c["HRatio"], c["kvHead"], c["use_compute_model"])
            plans.append(plan_fields(ki))
        return {"plans": plans, "tree": t}
    except Exception as exc:
        return {"raises": type(exc).__name__}


@pytest.fixture(scope="session")
def golden_small():
    return load_golden("plans_small.json.gz")


@pytest.fixture(scope="session")
def golden_large():
    return load_golden("plans_large.json.gz")


@pytest.fixture
def tuning():
    """Sets launch-geometry overrides of libpat_amd (pat_fwd_set_tuning) for one test:
    `tuning(direct_out=0)`; the automatic values come back when the test ends."""
    import ctypes as C
    from pat_amd import _lib, _prefix_attn
    lib = _lib.load()
    # the binding's measured geometry would take precedence over the process-wide overrides
    measured = _prefix_attn.get_autotune()
    _prefix_attn.set_autotune(False)

    def apply(**fields):
        t = _lib.FwdTuning.automatic()
        for name, value in fields.items():
            assert hasattr(t, name), name
            setattr(t, name, value)
        assert lib.pat_fwd_set_tuning(C.byref(t)) == 0

    yield apply
    auto = _lib.FwdTuning.automatic()
    lib.pat_fwd_set_tuning(C.byref(auto))
    _prefix_attn.set_autotune(measured)
