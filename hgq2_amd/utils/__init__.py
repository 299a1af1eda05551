from .minmax_trace import trace_minmax
from .models import qdense_mlp

__all__ = ['qdense_mlp', 'trace_minmax']
