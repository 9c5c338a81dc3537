from .btp import btp, btp_log

__all__ = ["btp", "btp_log"]
