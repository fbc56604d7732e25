"""MI355X-native (gfx950) fused LM-head log-probability path behind SkyRL's call signatures."""

__version__ = "0.1.0"
