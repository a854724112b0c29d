"""vllm_amd — MI355X (gfx950) implementation of vLLM's weight-only int4 "Marlin" operator surface.

Importing `vllm_amd.ops` loads the HIP shared library (built in-tree with `python -m vllm_amd.build`)
and registers the torch operators; nothing is imported eagerly here so that `import vllm_amd` works
in a build-only environment.
"""
__all__ = ["scalar_type"]
