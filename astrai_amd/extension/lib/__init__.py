"""Holds the built C-ABI library ``libastrai_w8a8.so`` (made by ``astrai_amd/csrc/Makefile``)."""
