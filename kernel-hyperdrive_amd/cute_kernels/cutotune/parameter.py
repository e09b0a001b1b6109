class CutoTuneParameter:
    """Sentinel default of a tunable argument: "let the tuner choose" (cute_kernels/cutotune/parameter.py:1)."""

    def __repr__(self) -> str:
        return "CutoTuneParameter()"
