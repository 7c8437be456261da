"""diopi_amd: an MI355X (gfx950) implementation of the DIOPI LLaMA-inference operators.

The product is ``diopi_amd/lib/libdiopi_impl.so`` (sources in ``diopi_amd/csrc``), a drop-in for
the reference's ``impl/lib/libdiopi_impl.so`` on this operator family.  The Python modules here are
the host-side mirror of the reference's conformance wrappers, calling that library through its C ABI:

* :mod:`diopi_amd.runtime`   - ctypes binding, Context / Tensor handles over torch memory
* :mod:`diopi_amd.functions` - rms_norm, rms_norm_backward, rotary_emb, destindex_copy_kv,
  token_attention, token_softmax_reducev, context_attention
"""
__all__ = ["runtime", "functions"]
