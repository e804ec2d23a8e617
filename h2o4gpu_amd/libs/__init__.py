"""Native-library bindings of the gfx950 k-means engine."""
