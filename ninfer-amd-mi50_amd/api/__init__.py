from .ninfer import Ninfer, Session

__all__ = ["Ninfer", "Session"]
