"""CPU oracle of the mHC layer path (test infrastructure; see naive_mhc.py and mhc_oracle.c)."""
