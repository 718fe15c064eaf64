"""Muscle moment-arm contractions behind the reference's entry points."""
