from .toolkit import gradient_check
