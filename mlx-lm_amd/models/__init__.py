"""Architectures: each module gives ``ModelArgs`` and ``Model``."""
