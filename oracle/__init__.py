"""TEST INFRASTRUCTURE: CPU oracles (see oracle/oracle.py).  Not importable from the product package."""
