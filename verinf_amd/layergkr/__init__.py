"""Stand-ins for the reference's `layergkr` modules on the Goldilocks hot path."""
