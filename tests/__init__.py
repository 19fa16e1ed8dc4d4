"""Test suite: CPU tests (oracle, config semantics, ABI, tuner loop) and GPU parity tests (marker gpu)."""
