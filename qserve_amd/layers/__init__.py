"""Building blocks of the served models: each mechanism takes its sizes and constants as parameters and runs through an
ops object (qserve_amd.layers.ops), so another model design can be composed from the same pieces."""
