"""CPU oracle of the TH FloatTensor semantics -- test infrastructure only."""
