"""GPT-2 inference engine for one AMD MI355X, in the manner of mlx-lm."""

__version__ = "0.1.0"
