"""MI355X-native batched Newton linear algebra (assemble H, tree / blocked L'DL,
solve) and muscle moment-arm contractions, behind the reference's entry points."""

__version__ = "0.1.0"
