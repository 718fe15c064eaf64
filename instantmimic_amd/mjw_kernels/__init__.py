"""Specialised solver kernels: structural eligibility, persistent scratch and
launchers, named like the reference's ``instantmimic.utils.mjw_kernels``."""
