"""Writes the golden data fixtures under tests/golden/ from data files the reference's
own tests hold.  Reads JSON / source text only; imports and runs nothing from the reference.

  moe_router_parity.json   logits -> route weights (top-k, renormalised) for the case in
                           tests/fixtures/moe_router_parity/unpacked_case.json with
                           num_experts / top_k from weights.json
  moe_expert_bank.json     hidden_gated, route_weights, trunk / expert weights and `mixed` of the same case
                           (tests/fixtures/moe_router_parity/unpacked_case.json, weights.json)
  e4m3_probe.json          the inputs and pinned bytes of tests/fp8_e4m3_probe.cu:23-27,55-56
  swiglu_probe.json        gate / up values of probes/public_kernel_probe.cu:55-60
"""
import json
import sys
from pathlib import Path

REF = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
OUT = Path(__file__).resolve().parent

fx = REF / "tests" / "fixtures" / "moe_router_parity"
weights = json.loads((fx / "weights.json").read_text())
cases = {}
for name in ("unpacked_case",):   # packed_case.json holds no logits (pooled-router path, out of scope)
    d = json.loads((fx / f"{name}.json").read_text())
    cases[name] = {"logits": d["logits"], "route_weights_pre_inhibition": d["route_weights_pre_inhibition"]}
(OUT / "moe_router_parity.json").write_text(json.dumps(
    {"num_experts": weights["num_experts"], "top_k": weights["top_k"], "cases": cases}, indent=1))

# the expert bank of the same case: gated hidden states, final route weights, trunk and expert weights, and the
# layer output `mixed` (data only; the pooled router that produced the route weights is out of scope)
d = json.loads((fx / "unpacked_case.json").read_text())
(OUT / "moe_expert_bank.json").write_text(json.dumps({
    "hidden_gated": d["hidden_gated"], "route_weights": d["route_weights"], "mixed": d["mixed"],
    "trunk_fc_in_w": weights["trunk_fc_in_w"], "trunk_fc_out_w": weights["trunk_fc_out_w"],
    "expert_fc_in_w": weights["expert_fc_in_w"], "expert_fc_out_w": weights["expert_fc_out_w"]}, indent=1))

# tests/fp8_e4m3_probe.cu:23-27 inputs, :55-56 pinned bytes (index -> byte)
(OUT / "e4m3_probe.json").write_text(json.dumps({
    "inputs": ["0.0", "-0.0", "1.0", "-1.0", "0.015625", "448.0", "-448.0", "447.0", "nan", "inf", "-inf"],
    "pinned": {"1": 0x80, "5": 0x7e, "6": 0xfe, "8": 0x7f, "9": 0x7f},
}, indent=1))

# probes/public_kernel_probe.cu:55-60, tolerance :29 region (close_enough 0.06)
(OUT / "swiglu_probe.json").write_text(json.dumps({
    "gate": [-2.0, -0.5, 0.5, 2.0], "up": [1.0, -2.0, 0.25, 3.0], "tolerance": 0.06}, indent=1))
print("fixtures written to", OUT)
