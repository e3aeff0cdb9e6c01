"""Model definitions.  Each module registers its class under the architecture name of its config.json
(qserve_amd.serving.registry)."""
