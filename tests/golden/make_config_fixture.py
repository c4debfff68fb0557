"""Writes tests/golden/sba_340m_config.json: the key/value pairs of the reference's model
configuration file, configs/sba_340m.json (16 values; a data file, read as JSON and written
back sorted).  Run in a container that holds the reference tree:

    python tests/golden/make_config_fixture.py [/root/reference]

The tests load the fixture through AutoConfig, so the shipped configuration class is held to
the reference's own configuration values rather than to a retyped copy of them.
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    with open(os.path.join(ref, "configs", "sba_340m.json")) as f:
        values = json.load(f)
    with open(os.path.join(HERE, "sba_340m_config.json"), "w") as f:
        json.dump(values, f, indent=1, sort_keys=True)
        f.write("\n")
    print(f"{len(values)} values written")


if __name__ == "__main__":
    main()
