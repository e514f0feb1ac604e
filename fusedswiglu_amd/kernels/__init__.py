"""Host launchers of the HIP kernels, one module per storage dtype like the reference's
fused_swiglu/kernels package."""
