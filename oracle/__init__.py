"""CPU oracle of the dropless-MoE hot path. Test infrastructure only; see `oracle/moe_oracle.py`."""
