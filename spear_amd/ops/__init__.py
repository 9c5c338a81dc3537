from .btp import btp, btp_log, phalanx_mix

__all__ = ["btp", "btp_log", "phalanx_mix"]
