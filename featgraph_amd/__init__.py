"""FeatGraph's SpMM / SDDMM hot path on MI355X (gfx950): hand-written HIP kernels in
``libfeatgraph_hip.so`` (built by ``python -m featgraph_amd.build``), called through its C ABI with ctypes.

``featgraph_amd.module``  -- the reference's ``featgraph.module`` surface (``VanillaSpMM*`` / ``VanillaSDDMM*``
                             with ``build()`` / ``run()``), plus the generalised operators;
``featgraph_amd.util``    -- ``util_convert_csr_to_dds`` / ``util_partition_adj_coo_2d``;
``featgraph_amd.autograd``-- ``Graph``: the same kernels as differentiable torch functions.

Importing the package loads nothing; the shared library is loaded on first use and its absence is an error.
"""
