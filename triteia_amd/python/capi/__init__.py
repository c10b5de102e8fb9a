from .marlin import mul_2_4, bmm_2_4, sbmm_2_4, sbmm_2_4_multilaunch
from .marlin import sbmm_2_4_routed, sbmm_2_4_planned, route_plan, routed_workspace
from .punica import add_lora_sgmv_cutlass, add_lora_bgmv, sgmv_routed

__all__ = ["mul_2_4", "bmm_2_4", "sbmm_2_4", "sbmm_2_4_multilaunch", "add_lora_sgmv_cutlass", "add_lora_bgmv",
           "sbmm_2_4_routed", "sbmm_2_4_planned", "route_plan", "routed_workspace", "sgmv_routed"]
