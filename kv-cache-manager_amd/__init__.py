"""A small, whole inference engine for one GPU (AMD MI355X, gfx950): from a model folder to
the next token.  Sub-packages: config, weights, parts, cache, engine, sampling, csrc."""
__version__ = "0.1.0"
