"""CPU oracle package (test infrastructure).  See mortar_oracle.py / mortar_oracle.c."""
