"""Command-line timing of the two operators, with the flags of the reference's benchmark scripts."""
