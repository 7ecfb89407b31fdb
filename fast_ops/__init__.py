"""Import-path compatibility: ``fast_ops.*`` resolves to the MI355X implementation in ``fast_ops_amd``."""
