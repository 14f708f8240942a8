from .layer import FusedMoE, FusedMoEConfig, KunlunUnquantizedFusedMoEMethod, SharedFusedMoE  # noqa: F401
