"""Generators: LEGO layouts in, HIP kernel text out (one module per kernel family)."""
