"""Helpers for tests written against this package (the role of ``theano/tests``)."""
