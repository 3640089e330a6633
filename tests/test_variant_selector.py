"""The rule matcher of cut_amd/variant_selector.py against the semantics of the reference's
VariantSelector::select (runtime/VariantSelector.cpp:380-428): first match wins, exact shape and / or a half-open
range of total elements, backend-specific entry before the backend-agnostic one, caller's default when nothing is
loaded or no entry exists.  CPU only."""
import json

from cut_amd.variant_selector import VariantSelector

DATA = {"operators": {
    "MatMul": {
        "default_variant": 7,
        "rules": [{"variant": 9, "conditions": {"total_elements_max": 100}}],
        "backends": {
            "hip": {"default_variant": 3, "rules": [
                {"variant": 5, "conditions": {"shape": [2048, 4096, 14336]}},
                {"variant": 4, "conditions": {"total_elements_min": 1000, "total_elements_max": 2000}},
                {"variant": 1, "conditions": {"shape": [2, 10, 150], "total_elements_min": 5000}},
                {"variant": 2, "conditions": {"total_elements_min": 1200}},
            ]},
            "cuda": {"default_variant": 11, "rules": []},
        }},
    "Scan": {"default_variant": 1},
}}


def make(tmp_path):
    p = tmp_path / "tuning_data.json"
    p.write_text(json.dumps(DATA))
    s = VariantSelector()
    assert s.load(str(p))
    return s


def test_unloaded_returns_the_callers_default(tmp_path):
    s = VariantSelector()
    assert s.select("MatMul", [1, 2, 3], 42) == 42
    assert not s.load(str(tmp_path / "missing.json")) and not s.loaded
    (tmp_path / "bad.json").write_text("[1, 2]")
    assert not s.load(str(tmp_path / "bad.json"))


def test_first_match_wins_and_ranges_are_half_open(tmp_path):
    s = make(tmp_path)
    assert s.select("MatMul", [2048, 4096, 14336], 0, "hip") == 5          # exact shape
    assert s.select("MatMul", [10, 10, 10], 0, "hip") == 4                  # 1000 is inside [1000, 2000)
    assert s.select("MatMul", [10, 10, 12], 0, "hip") == 4                  # 1200: the earlier rule wins over variant 2
    assert s.select("MatMul", [10, 10, 20], 0, "hip") == 2                  # 2000 is outside [1000, 2000)
    assert s.select("MatMul", [2, 10, 150], 0, "hip") == 2                  # shape matches but 3000 < its minimum of 5000
    assert s.select("MatMul", [3, 3, 3], 0, "hip") == 3                     # no rule: the entry's default
    assert s.select("MatMul", [4096, 2048, 14336], 0, "hip") == 2           # same total, other shape: not the exact rule


def test_backend_preference_and_fallbacks(tmp_path):
    s = make(tmp_path)
    assert s.select("MatMul", [3, 3, 3], 0, "cuda") == 11
    assert s.select("MatMul", [3, 3, 3], 0, "vulkan") == 9                  # no such backend: the agnostic entry (27 < 100)
    assert s.select("MatMul", [30, 30, 30], 0, "") == 7
    assert s.select("Scan", [5], 0, "hip") == 1
    assert s.select("Transpose", [5, 5], 6, "hip") == 6                     # no entry at all


def test_committed_hip_section_is_well_formed():
    import os
    from cut_amd import variant_selector as vs
    if not os.path.exists(vs.DEFAULT_PATH):
        import pytest
        pytest.skip("no tuning_data.json committed")
    s = VariantSelector()
    assert s.load(vs.DEFAULT_PATH)
    data = json.load(open(vs.DEFAULT_PATH))
    nvar = len(data["variant_names"])
    for name, entry in s.operators.items():
        assert name.endswith("@hip")
        assert entry["default"] == -1
        for r in entry["rules"]:
            assert 0 <= r["variant"] < nvar and len(r["shape"]) == 3
