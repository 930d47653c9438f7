"""TEST INFRASTRUCTURE ONLY: CPU oracle of the BCPNN layer step (see bcpnn_oracle.c, oracle.py)."""
