from .training_context import TrainingContext, execute_backward_pass, execute_forward_pass, forward_context

__all__ = ["TrainingContext", "execute_forward_pass", "execute_backward_pass", "forward_context"]
