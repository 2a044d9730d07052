"""enzyme_ad: MI355X-native stand-in for the reference's `enzyme_ad` package
(reference: src/enzyme_ad/__init__.py).  Only `enzyme_ad.jax` exists."""
