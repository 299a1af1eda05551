from .callbacks import BaseBetaPID, BetaPID, BetaScheduler, Callback, FreeEBOPs, PID, PieceWiseSchedule, fit

__all__ = ['BetaPID', 'BaseBetaPID', 'BetaScheduler', 'PieceWiseSchedule', 'FreeEBOPs', 'PID', 'Callback', 'fit']
