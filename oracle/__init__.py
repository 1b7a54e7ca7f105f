"""Test oracle (CPU).  TEST INFRASTRUCTURE ONLY — the library never imports this package."""
