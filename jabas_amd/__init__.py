"""MI355X-native per-GPU gradient synchronisation for IIDP/JABAS: batch-weighted VSW
aggregate + gradient statistics + fused optimizer, behind the reference's hook surface."""
__version__ = "0.1.0"
