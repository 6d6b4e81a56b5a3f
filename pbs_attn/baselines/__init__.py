"""Baselines of the reference that this build provides: the un-permuted MeanPooling method."""
