"""CPU oracle of the CatBoost evaluation path. Test infrastructure only."""
