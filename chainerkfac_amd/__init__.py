"""MI355X-native K-FAC per-layer hot path behind the chainerkfac API."""
from chainerkfac_amd import communicators  # NOQA
