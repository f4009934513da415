"""Parity oracle for the SGNS hot path: test infrastructure, never imported by the product."""
