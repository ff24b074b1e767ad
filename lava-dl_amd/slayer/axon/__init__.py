from .delay import delay, Delay

__all__ = ['delay', 'Delay']
