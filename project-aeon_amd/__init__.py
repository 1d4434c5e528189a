"""MI355X-native routed-expert hot path for project-aeon (see include/aeon_mi355.h)."""
