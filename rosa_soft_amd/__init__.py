"""MI355X-native rosa_soft training operators (package surface is filled in below)."""
