from .experts import MoEExperts, MoEExpertsFP8, MoEExpertsSerial

__all__ = ["MoEExperts", "MoEExpertsSerial", "MoEExpertsFP8"]
