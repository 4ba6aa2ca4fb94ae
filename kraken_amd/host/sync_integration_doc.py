"""Copies the adapters of kraken_ref_tables.h (between its integration markers) into the
repository's integration notes, between that document's own markers, so that it prints the code
that is compiled against the reference's interface and not a second typing of it.

    python kraken_amd/host/sync_integration_doc.py
"""
import os

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
BEGIN, END = "<!-- adapters:begin -->", "<!-- adapters:end -->"


def main():
    src = open(os.path.join(HERE, "kraken_ref_tables.h")).read()
    body = src[src.index("// [integration:begin]") + len("// [integration:begin]"):src.index("// [integration:end]")]
    path = os.path.join(ROOT, "INTEGRATION.md")
    doc = open(path).read()
    a, b = doc.index(BEGIN) + len(BEGIN), doc.index(END)
    doc = doc[:a] + "\n```cpp\n" + body.strip() + "\n```\n" + doc[b:]
    open(path, "w").write(doc)


if __name__ == "__main__":
    main()
