"""Mirror of the reference's package layout for the MXFP4 scaled-GEMM path:
``wave_lang.kernel.X`` -> ``wave_amd.kernel.X`` for the modules a user of
that path imports (lang, wave.compile, wave.constraints, wave.templates,
wave.schedules, wave.utils.mxfp_utils)."""
