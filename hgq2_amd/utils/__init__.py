from .models import qdense_mlp

__all__ = ['qdense_mlp']
