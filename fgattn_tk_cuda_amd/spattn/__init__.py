"""Mirror of the reference's ``spattn`` package on top of the gfx950 library.

``spattn.cuda_attn`` is the compiled operator extension (it registers
``torch.ops.cuda_attn.*``); ``spattn.mask_utils`` and
``spattn.sparseattn_functionals`` carry the reference's Python-level helpers.
Put the parent directory of this package on ``sys.path`` to import it as ``spattn``.
"""
