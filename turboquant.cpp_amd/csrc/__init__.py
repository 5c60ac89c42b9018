"""HIP sources for gfx950, their build, and their Python face (``ops``)."""
