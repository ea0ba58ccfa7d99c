"""Generator of schema_generated.h and schema_names.cpp: derives flatbuffer field slot numbers, enum values and operation
names from the .fbs schema text of a tt-mlir checkout (the wire-format contract,
include/ttmlir/Target/{Common,TTNN}/**/*.fbs).

    python gen_schema.py <tt-mlir checkout> [output directory]     (default output: the directory of this file)

There is no flatc in this build, so the reader / writer in flatbuffer.h works from these constants.  Regenerate when the
schemas of the tt-mlir revision to be served change; tests/test_runtime_host.py checks that the committed files are what
this script makes of the checkout at hand."""
import os
import re
import sys

C_TYPES = {"uint": "uint32_t", "uint32": "uint32_t", "uint16": "uint16_t", "ushort": "uint16_t", "uint8": "uint8_t",
           "ubyte": "uint8_t", "int8": "int8_t"}


def schema_files(target_dir):
    files = ["Common/types.fbs", "Common/version.fbs", "Common/debug_info.fbs", "TTNN/types.fbs", "TTNN/binary.fbs",
             "TTNN/program.fbs"]
    return files + ["TTNN/operations/" + f for f in sorted(os.listdir(os.path.join(target_dir, "TTNN", "operations")))]


def parse(target_dir):
    """(unions, enums, tables) of the schema files: member lists in declaration order."""
    unions, enums, tables = {}, {}, {}
    for f in schema_files(target_dir):
        text = re.sub(r"//[^\n]*", "", open(os.path.join(target_dir, f)).read())
        for m in re.finditer(r"\bunion\s+(\w+)\s*\{([^}]*)\}", text):
            unions[m.group(1)] = [x.strip().split(":")[0].strip() for x in m.group(2).split(",") if x.strip()]
        for m in re.finditer(r"\benum\s+(\w+)\s*:\s*(\w+)\s*(\([^)]*\))?\s*\{([^}]*)\}", text):
            values, nxt = [], 0
            for x in m.group(4).split(","):
                x = x.strip()
                if not x:
                    continue
                if "=" in x:
                    name, v = [y.strip() for y in x.split("=")]
                    nxt = int(v)
                else:
                    name = x
                values.append((name, nxt))
                nxt += 1
            enums[m.group(1)] = (m.group(2), values)
        for m in re.finditer(r"\btable\s+(\w+)\s*\{([^}]*)\}", text):
            fields = []
            for x in m.group(2).split(";"):
                x = x.strip()
                if not x:
                    continue
                name, ty = x.split(":", 1)
                fields.append((name.strip(), ty.split("=")[0].strip().split("(")[0].strip()))
            tables[m.group(1)] = fields
    return unions, enums, tables


def generate(ref_root):
    """{file name: text} for schema_generated.h and schema_names.cpp."""
    unions, enums, tables = parse(os.path.join(ref_root, "include", "ttmlir", "Target"))
    out = ["// Field slot numbers and enum values of the TTNN flatbuffer schema (the wire-format contract",
           "// between the tt-mlir compiler and a runtime): include/ttmlir/Target/{Common,TTNN}/**/*.fbs.",
           "// Slots are implicit in the schema: declaration order, a union field taking two slots",
           "// (<name>_type then <name>).  Generated from the schema text; do not edit by hand.",
           "#pragma once", "#include <cstdint>", "", "namespace ttmlir_amd::schema {", ""]
    for name, (base, values) in sorted(enums.items()):
        out.append("enum class %s : %s {" % (name, C_TYPES[base]))
        out += ["  %s = %d," % (n, v) for n, v in values]
        out.append("};")
    for name, members in sorted(unions.items()):
        out.append("enum class %s : uint8_t {" % name)
        out.append("  NONE = 0,")
        out += ["  %s = %d," % (n.split(".")[-1], i + 1) for i, n in enumerate(members)]
        out.append("};")
    out.append("")
    for name, fields in sorted(tables.items()):
        out.append("struct %s {" % name)
        out.append("  enum : int {")
        slot = 0
        for n, ty in fields:
            if ty.strip("[]").split(".")[-1] in unions and not ty.startswith("["):
                out.append("    f_%s_type = %d," % (n, slot))
                slot += 1
            out.append("    f_%s = %d," % (n, slot))
            slot += 1
        out.append("    kNumFields = %d" % slot)
        out.append("  };")
        out.append("};")
    out.append("")
    out.append("const char *opTypeName(OpType t);")
    out.append("}  // namespace ttmlir_amd::schema")
    names = ["  case OpType::%s: return \"%s\";" % (n, n) for n in unions["OpType"]]
    names_cpp = ("// OpType names (union member order of include/ttmlir/Target/TTNN/program.fbs:36-170).  Generated.\n"
                 "#include \"schema_generated.h\"\n\nnamespace ttmlir_amd::schema {\nconst char *opTypeName(OpType t) {\n"
                 "  switch (t) {\n  case OpType::NONE: return \"NONE\";\n" + "\n".join(names) +
                 "\n  }\n  return \"?\";\n}\n}  // namespace ttmlir_amd::schema\n")
    return {"schema_generated.h": "\n".join(out) + "\n", "schema_names.cpp": names_cpp}


if __name__ == "__main__":
    if len(sys.argv) < 2:
        raise SystemExit(__doc__)
    outdir = sys.argv[2] if len(sys.argv) > 2 else os.path.dirname(os.path.abspath(__file__))
    for fname, text in generate(sys.argv[1]).items():
        with open(os.path.join(outdir, fname), "w") as fh:
            fh.write(text)
        print("wrote", os.path.join(outdir, fname))
