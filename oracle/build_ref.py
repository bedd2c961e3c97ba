"""Compiles the reference's own host sources, where they lie, into oracle/_ref/ (a checker only).
Placeholder until the recipe is written: reports that nothing was built."""
import sys
print("oracle/_ref: no recipe yet for", sys.argv[1:])
