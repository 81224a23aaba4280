"""CPU oracle for kraken_amd — TEST INFRASTRUCTURE ONLY (see oracle/oracle.py)."""
