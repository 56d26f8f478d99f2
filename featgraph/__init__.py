"""Import-path alias: ``featgraph.module`` / ``featgraph.util`` resolve to the gfx950
implementation in ``featgraph_amd`` so call sites written for the reference package keep
their imports."""
