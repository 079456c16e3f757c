"""MI355X-native bitfield-masked attention behind Cornstarch's kernel API."""

__version__ = "0.1.0"
