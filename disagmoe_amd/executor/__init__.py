from .executor import ExpertsExecutor

__all__ = ["ExpertsExecutor"]
