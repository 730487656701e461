"""Writes engine_sidecar_symbols.json: the symbols the reference's resident engine binds from
its tile-ops sidecar, and whether it requires each (tile_.require<...>) or can do without
(tile_.optional<...>), read from the text of
neuralfn/csrc/native_gpt2/resident_glimmer_cuda.cpp in the reference checkout.  Symbols bound
by enable_vision() (only when a vision companion is loaded) are listed apart from those the
runtime's constructor binds for text decoding.

Run where the reference checkout exists: python tests/golden/make_engine_symbol_list.py
"""
import json
import re
from pathlib import Path

SOURCE = Path("/root/reference/neuralfn/csrc/native_gpt2/resident_glimmer_cuda.cpp")
TARGET = Path(__file__).resolve().parent / "engine_sidecar_symbols.json"


def main() -> None:
    text = SOURCE.read_text()
    pattern = r"tile_\.(require|optional)<[A-Za-z0-9_]+>\(\s*\"([a-z0-9_]+)\"\s*\)"
    cut = text.index("void enable_vision()")
    decode, vision = re.findall(pattern, text[:cut]), re.findall(pattern, text[cut:])
    symbols = {"required": sorted({name for kind, name in decode if kind == "require"}),
               "optional": sorted({name for kind, name in decode if kind == "optional"}),
               "vision_required": sorted({name for kind, name in vision if kind == "require"}),
               "vision_optional": sorted({name for kind, name in vision if kind == "optional"})}
    TARGET.write_text(json.dumps(symbols, indent=1) + "\n")
    print({kind: len(names) for kind, names in symbols.items()}, "->", TARGET)


if __name__ == "__main__":
    main()
