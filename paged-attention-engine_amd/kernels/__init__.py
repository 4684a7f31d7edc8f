"""Python side of the gfx950 kernel library: building it and calling into it."""
