"""MI355X-native Float8Linear hot path behind float8_experimental's Python API."""
