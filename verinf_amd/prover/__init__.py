"""Stand-ins for the reference's `prover` modules on the Goldilocks hot path."""
