"""Drop-in for the reference's pybind module `custom_esimd_kernels_sglang.moe_grouped_gguf_xpu`
(sglang/custom-esimd-kernels/csrc/moe_grouped/moe_grouped_entry.sycl:108-127): grouped K-quant MoE GEMMs
over chunks {expert, first row, rows} of expert-sorted routes, same names, argument order and defaults."""
from mi355x_qlinear.ops import moe_down_q5k_ggemv, moe_down_q6k_ggemv, moe_up_q4k_ggemv  # noqa: F401
