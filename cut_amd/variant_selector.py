"""Shape -> kernel-variant rules, the reference's VariantSelector (runtime/VariantSelector.cpp:283-428) for the
"hip" backend.

Same file format and the same matching: `{"operators": {<op>: {"backends": {<backend>: {"default_variant": d,
"rules": [{"variant": v, "conditions": {"shape": [M, K, N]}} | {"variant": v, "conditions":
{"total_elements_min": a, "total_elements_max": b}}]}}}}}`; the first rule that matches wins (exact shape,
dimension for dimension, and/or `a <= prod(shape) < b`), then the entry's default variant; a backend-specific entry is
preferred to a backend-agnostic one (rules directly under the operator); without any entry the caller's default is
returned.  `cut_amd/tuning_data.json` holds the "hip" section measured by `cut_amd/autotune.py` on an MI355X.
"""
import json
import math
import os

BACKEND = "hip"
DEFAULT_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tuning_data.json")


class VariantSelector:
    def __init__(self):
        self.operators = {}
        self.loaded = False

    @staticmethod
    def _key(op: str, backend: str) -> str:
        return f"{op}@{backend}" if backend else op

    @staticmethod
    def _parse_rules(obj: dict) -> dict:
        dv = obj.get("default_variant", 0)
        rules = []
        for rv in obj.get("rules", []) if isinstance(obj.get("rules", []), list) else []:
            cond = rv.get("conditions", {}) if isinstance(rv.get("conditions", {}), dict) else {}
            rules.append({"variant": int(rv.get("variant", 0)),
                          "min": int(cond.get("total_elements_min", -1)),
                          "max": int(cond.get("total_elements_max", -1)),
                          "shape": [int(v) for v in cond.get("shape", [])]})
        return {"default": int(dv) if isinstance(dv, (int, float)) else 0, "rules": rules}

    def load(self, path: str = DEFAULT_PATH) -> bool:
        """False (and nothing changes) when the file is missing or is not a tuning file."""
        try:
            with open(path) as fh:
                root = json.load(fh)
        except (OSError, ValueError):
            return False
        ops = root.get("operators") if isinstance(root, dict) else None
        if not isinstance(ops, dict):
            return False
        table = {}
        for name, val in ops.items():
            if not isinstance(val, dict):
                continue
            for backend, sub in (val.get("backends") or {}).items():
                if isinstance(sub, dict):
                    table[self._key(name, backend)] = self._parse_rules(sub)
            if "default_variant" in val or "rules" in val:
                table[name] = self._parse_rules(val)
        self.operators = table
        self.loaded = True
        return True

    def select(self, op: str, shape, default_variant: int, backend: str = BACKEND) -> int:
        if not self.loaded:
            return default_variant
        shape = [int(v) for v in shape]
        total = math.prod(shape)

        def evaluate(entry):
            for r in entry["rules"]:
                shape_ok = not r["shape"] or r["shape"] == shape
                min_ok = r["min"] < 0 or total >= r["min"]
                max_ok = r["max"] < 0 or total < r["max"]
                if shape_ok and min_ok and max_ok:
                    return r["variant"]
            return entry["default"]

        if backend and self._key(op, backend) in self.operators:
            return evaluate(self.operators[self._key(op, backend)])
        if op in self.operators:
            return evaluate(self.operators[op])
        return default_variant


_instance = VariantSelector()


def instance() -> VariantSelector:
    return _instance
