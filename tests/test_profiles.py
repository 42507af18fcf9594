"""The tracked traffic table (profiles/traffic.json) names the instance each figure was profiled on; it must be the
instance the tuned records yield today, and the profile summary it points at must exist (no GPU needed)."""
import json
import os

from heron_amd import tuned

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_traffic_table_matches_tuned_instances():
    table = json.load(open(os.path.join(ROOT, "profiles", "traffic.json")))
    rows = {k: v for k, v in table.items() if not k.startswith("_")}
    assert rows
    for name, row in rows.items():
        assert name in tuned.CASES, name
        assert row["instance"] == list(tuned.load(name).desc.as_tuple()), "re-profile %s: its tuned instance changed" % name
        assert os.path.exists(os.path.join(ROOT, row["profile"])), row["profile"]
        assert abs(row["bytes"] - (row["fetch_kib"] * 2.0 + row["write_kib"]) * 1024) < 1.0
