"""The interface mirror (raf_amd/csrc/dialect/raf_iface.h) against the text of the reference's
headers.  The `hip` dialect is written against the mirror because RAF itself cannot be compiled
here; this test ties every declaration the dialect relies on to the reference, so that the mirror
cannot drift: each declaration below must occur, white space aside, in the reference header AND in
the mirror.  Where the mirror names an operator by its string name instead of an `ir::Op` (there is
no TVM operator registry here) the pair gives both spellings.

Needs the reference tree: skipped where /root/reference is absent (the GPU box)."""
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
REFERENCE = Path("/root/reference")
MIRROR = ROOT / "raf_amd" / "csrc" / "dialect" / "raf_iface.h"

pytestmark = pytest.mark.skipif(not (REFERENCE / "include" / "raf" / "op.h").exists(),
                                reason="the reference tree is not present")


def squeeze(text: str) -> str:
    """Comments out, all white space out."""
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    text = text.replace("\\\n", " ")  # macro continuation lines
    return re.sub(r"\s+", "", text)


def lines(path: Path, first: int, last: int) -> str:
    return "\n".join(path.read_text().splitlines()[first - 1:last])


# (reference header, first line, last line, declaration there, declaration in the mirror or None for "the same")
OP_H = REFERENCE / "include" / "raf" / "op.h"
DIALECT_H = REFERENCE / "include" / "raf" / "dialect.h"
DECLARATIONS = [
    # OpEnv, include/raf/op.h:59-105
    (OP_H, 59, 105, "virtual std::string name() const = 0;", None),
    (OP_H, 59, 105, "virtual void Execute(const CallValues& call) = 0;", None),
    (OP_H, 59, 105, "virtual void Execute(const std::vector<value::Value>& inputs, value::Value output) = 0;", None),
    (OP_H, 59, 105, "std::vector<std::string> error_msgs;", None),
    (OP_H, 59, 105, "bool HasError() { return !error_msgs.empty(); }", None),
    (OP_H, 59, 105, "void RequestWorkspace(void** dest, const Device& device, int64_t nbytes);", None),
    (OP_H, 59, 105, "void RequestStream(void** dest, const Device& device, int tag_idx);", None),
    (OP_H, 59, 105, "std::vector<int> arg_indices;", None),
    (OP_H, 59, 105, "static void SetStreamForAllBackends(Device device, void* stream);", None),
    (OP_H, 59, 110, "using OpEnvPtr = std::shared_ptr<OpEnv>;", None),
    # OpEnvMaker, include/raf/op.h:107-150
    (OP_H, 107, 150, "using FMakeOpEnv = std::function<OpEnv*(const CallValues& call)>;", None),
    (OP_H, 107, 150, "OpEnvMaker& set_name(const std::string& name);", "OpEnvMaker& set_name(const std::string& n)"),
    (OP_H, 107, 150, "OpEnvMaker& set_func(FMakeOpEnv f);", "OpEnvMaker& set_func(FMakeOpEnv f)"),
    (OP_H, 107, 150, "OpEnv* operator()(const CallValues& call) const", None),
    (OP_H, 107, 150, "static const OpEnvMaker* Get(const std::string& op_name);", None),
    (OP_H, 107, 150, "std::string name;", None),
    # Dialect, include/raf/dialect.h:60-104
    (DIALECT_H, 60, 104, "Dialect& set_enable(DevType device_type);", None),
    (DIALECT_H, 60, 104, "bool is_enabled(DevType device_type) const;", None),
    (DIALECT_H, 60, 104, "static const Dialect* Get(const std::string& dialect_name);", None),
    (DIALECT_H, 60, 104, "static bool IsEnabled(const std::string& dialect, DevType device_type);", None),
    (DIALECT_H, 60, 104, "static std::vector<std::string> GetEnabledDialects(DevType device_type);", None),
    # OpDialect, include/raf/dialect.h:106-170
    (DIALECT_H, 106, 170, "std::string dialect;", None),
    (DIALECT_H, 106, 170, "std::string dialect_op;", None),
    (DIALECT_H, 106, 170, "int plevel;", None),
    (DIALECT_H, 106, 170, "using TDialectList = std::list<DialectOpEntry>;", None),
    (DIALECT_H, 106, 170, "OpDialect& set_name(const std::string& name);", "OpDialect& set_name(const std::string& n)"),
    (DIALECT_H, 106, 170,
     "OpDialect& add_dialect(const std::string& dialect_name, const std::string& dialect_op, int plevel = 10);", None),
    (DIALECT_H, 106, 170, "static TDialectList GetDispatchList(const ir::Op& op, DevType device_type);",
     "static TDialectList GetDispatchList(const std::string& base_op, DevType device_type);"),
    (DIALECT_H, 106, 170,
     "static ir::Op Dispatch(const ir::Op& base_op, DevType device_type, const std::vector<std::string>& skip_dialects = {});",
     "static std::string Dispatch(const std::string& base_op, DevType device_type, "
     "const std::vector<std::string>& skip_dialects = {});"),
    (DIALECT_H, 106, 170, "static ir::Op Lower(const ir::Op& base_op, const std::string& dialect);",
     "static std::string Lower(const std::string& base_op, const std::string& dialect);"),
    (DIALECT_H, 106, 170, "TDialectList dialect_ops_;", None),
    # helpers, include/raf/dialect.h:199-217
    (DIALECT_H, 199, 217, "bool IsDialectOp(const ir::Op& op);", "bool IsDialectOp(const std::string& op);"),
    (DIALECT_H, 199, 217, "std::string GetDialect(const ir::Op& op);", "std::string GetDialect(const std::string& op);"),
    (DIALECT_H, 199, 217, "ir::Op GetBaseOp(const ir::Op& dialect_op);", "std::string GetBaseOp(const std::string& op);"),
    # registration macros, include/raf/dialect.h:222-243 and include/raf/op.h:326-334
    (DIALECT_H, 222, 243, "#define RAF_BASE_OP_NAME(NAME)", None),
    (DIALECT_H, 222, 243, "#define RAF_DIALECT_OP_NAME(DIALECT, NAME)", None),
    (DIALECT_H, 222, 243, "#define RAF_REGISTER_DIALECT(DIALECT_NAME)", None),
    (DIALECT_H, 222, 243, ".set_name(DIALECT_NAME)", None),
    (DIALECT_H, 222, 243, "#define RAF_REGISTER_DIALECT_OP(DIALECT, OP, PLEVEL)", None),
    (DIALECT_H, 222, 243, ".add_dialect(#DIALECT, RAF_DIALECT_OP_NAME(DIALECT, OP), PLEVEL)",
     "RegisterDialectOp_(#DIALECT, RAF_BASE_OP_NAME(OP), RAF_DIALECT_OP_NAME(DIALECT, OP), PLEVEL)"),
    (DIALECT_H, 222, 243, "(raf.op.DIALECT.NAME)", None),
    (OP_H, 320, 340, "#define RAF_OP_ENV_MAKER(OP_NAME, FOP_ENV_MAKER)", None),
    (OP_H, 320, 340, ".set_name(OP_NAME).set_func(FOP_ENV_MAKER)", None),
]


@pytest.mark.parametrize("header,first,last,theirs,ours", DECLARATIONS,
                         ids=[f"{d[0].name}:{d[3][:48]}" for d in DECLARATIONS])
def test_declaration_is_in_the_reference_and_in_the_mirror(header, first, last, theirs, ours):
    assert squeeze(theirs) in squeeze(lines(header, first, last)), \
        f"{header}:{first}-{last} no longer declares `{theirs}`: the reference moved; update the mirror and this table"
    want = ours or theirs
    assert squeeze(want) in squeeze(MIRROR.read_text()), f"raf_iface.h does not declare `{want}`"


def test_the_dialect_uses_nothing_the_table_does_not_pin():
    """Every member of OpEnv / OpEnvMaker / Dialect / OpDialect that hip_dialect.cc touches is one of
    the declarations above (or one of the mirror's two accessors for recorded requests)."""
    src = (ROOT / "raf_amd" / "csrc" / "dialect" / "hip_dialect.cc").read_text()
    used = set(re.findall(r"\b(RequestWorkspace|RequestStream|RequestDistributed|BindExecutor|GetRequests|"
                          r"arg_indices|error_msgs|HasError|SetStreamForAllBackends)\b", src))
    pinned = squeeze(" ".join(d[3] for d in DECLARATIONS))
    for name in used:
        assert name in pinned, f"hip_dialect.cc uses OpEnv::{name}, which no row of the table pins"
    code = re.sub(r"//[^\n]*", "", src)  # macros named in comments (citations of the reference) do not count
    for macro in set(re.findall(r"\b(RAF_[A-Z_]+)\(", code)) - {"RAF_CHECK"}:
        assert macro in pinned, f"hip_dialect.cc uses {macro}, which no row of the table pins"


def test_stream_tags_are_the_reference_s():
    """The two copy-stream tags the fuse / defuse OpEnvs request."""
    pool = (REFERENCE / "include" / "raf" / "stream_pool.h").read_text()
    mirror = squeeze(MIRROR.read_text())
    for value, name in ((5, "MemCpyCudaToCuda1"), (6, "MemCpyCudaToCuda2"), (1, "CudaCompute")):
        assert re.search(rf"ENUM_DEF_ENTRY_WITH_NAME\(StreamTagEnum,\s*{value},\s*\w+,\s*k{name},", pool), name
        assert f"k{name}={value}," in mirror, name
    memory = (REFERENCE / "src" / "op" / "dialect" / "cuda" / "memory.cc").read_text()
    assert "RequestStream(&stream, cv->device, StreamTagEnum::MemCudaToCuda1());" in memory
    assert "RequestStream(&stream, cv->device, StreamTagEnum::MemCudaToCuda2());" in memory
