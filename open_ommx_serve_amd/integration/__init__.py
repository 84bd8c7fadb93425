"""Serving-engine seams over the OMMX decode-attention operators.

Mirrors ``ommx_gpu_serve.integration`` of the reference for the part that feeds the hot path:
the per-step host seam (request slots, window lengths, fixed-address step buffers) and the
attention-backend surface that calls the store and decode operators.
"""
