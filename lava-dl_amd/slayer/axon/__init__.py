from .delay import delay, Delay
from .delta import Delta

__all__ = ['delay', 'Delay', 'Delta']
