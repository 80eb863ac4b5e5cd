from . import mem_eff_attention  # noqa: F401  (registers the rocm.mem_eff_attention.* hooks)
