// horizontal-fuser -- source-to-source front end: two GPU kernels + a split config in, ONE
// fused HIP kernel for gfx950 out.
//
// Same command line and file contract as the reference's tool
// (horizontal-fuser/src/main.cc:20-32,79-96; drivers Fuse.cc:64-221 bfuse, :223-376 hfuse):
//
//   horizontal-fuser [-h] [-b] [-y yaml_output] [-o output] fusion_config kernel_config compile_commands
//
//     fusion_config    fusions.yaml : sequence of {File, Kernels}          (Utils.h:82-90)
//     kernel_config    kernels.yaml : map name -> KernelInfo              (Utils.h:70-80)
//     compile_commands directory holding the kernel source named by File  (Fuse.cc:82-84)
//   outputs  <output>/<K1>_<K2>_{bfuse,hfuse}.hip  and  <yaml_output>/{bfuse,hfuse}_kernels.yaml
//            (Fuse.cc:203-220, :359-375; the reference writes .cu)
//
// Extensions, all optional: -p zigzag|proportional|chunked|ranges (block pattern, default the
// reference's live zig-zag), -M/-N (zig-zag ratio cap and multiplier), -c (chunk / min-option),
// -w (thread-range padding, default 64 = one gfx950 wavefront; 32 reproduces the reference).
//
// What the reference does with nine Clang libTooling passes over the AST (Tools.cc:68-290,
// Matchers.cc) is done here on the token stream of the two kernels, which is enough for the
// C subset TVM emits and for hand-written kernels in the same style:
//   * parameters p of kernel K are renamed K_p_                      (Tools.cc:100-135)
//   * blockIdx/threadIdx/blockDim/gridDim .x/.y/.z become locals blockIdx_x_ ...
//                                                                     (Matchers.cc:255-286)
//   * bfuse: static __shared__ arrays move into struct K inside `union ShrdUnion`, accesses
//     become SU_.K.name                                               (Tools.cc:199-258)
//   * hfuse: __shared__ arrays stay per branch (LDS = sum); __syncthreads() becomes a
//     barrier over that side's wavefronts only.  CUDA's `bar.sync id, n` (Matchers.cc:288-320)
//     has no gfx950 counterpart, so the emitted code carries a small LDS arrival-counter
//     barrier (bfuse_side_barrier) instead.
//   * the dispatch prologue is generated from the same index maps as the runtime
//     (dispatch.h), printed as the reference's if / else-if chain     (Algorithms.cc)
// The input file is never modified (the reference rewrites it in place and restores it).
#include <getopt.h>

#include <algorithm>
#include <cctype>
#include <cstdio>
#include <cstring>
#include <filesystem>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <map>
#include <set>
#include <sstream>
#include <string>
#include <vector>

#include "../dispatch.h"

using namespace std;
using namespace bfuse;

namespace {

[[noreturn]] void die(const string& msg)
{
    // the reference exits with status 0 on every error (Fuse.cc:87-91); a failing tool should say so
    cerr << "horizontal-fuser: error: " << msg << "\n";
    exit(1);
}

string read_file(const string& path)
{
    ifstream in(path);
    if (!in) die("cannot open " + path);
    stringstream ss;
    ss << in.rdbuf();
    return ss.str();
}

void write_file(const string& dir, const string& name, const string& text)
{
    std::error_code ec;
    std::filesystem::create_directories(dir, ec);
    ofstream out(dir + "/" + name);
    if (!out) die("cannot write " + dir + "/" + name);
    out << text;
}

// ---- minimal YAML (block style: maps, "- " sequences, scalars), as written by PyYAML and llvm::yaml
struct Line {
    int indent;
    bool dash;      // starts with "- "
    string key;     // empty for a bare sequence scalar
    string value;   // may be empty (nested block follows)
};

string trim(const string& s)
{
    size_t a = s.find_first_not_of(" \t\r\n"), b = s.find_last_not_of(" \t\r\n");
    return a == string::npos ? "" : s.substr(a, b - a + 1);
}

vector<Line> yaml_lines(const string& text)
{
    vector<Line> out;
    stringstream ss(text);
    string raw;
    while (getline(ss, raw)) {
        size_t hash = raw.find(" #");
        if (hash != string::npos) raw = raw.substr(0, hash);
        if (trim(raw).empty() || trim(raw) == "---" || trim(raw) == "...") continue;
        if (trim(raw)[0] == '#') continue;
        Line l{};
        l.indent = (int)raw.find_first_not_of(' ');
        string body = trim(raw);
        if (body.rfind("- ", 0) == 0 || body == "-") {
            l.dash = true;
            l.indent += 2;
            body = body.size() > 1 ? trim(body.substr(2)) : "";
        }
        size_t colon = body.find(':');
        if (colon != string::npos && (colon + 1 == body.size() || body[colon + 1] == ' ')) {
            l.key = trim(body.substr(0, colon));
            l.value = trim(body.substr(colon + 1));
        } else {
            l.value = body;
        }
        auto unq = [](string& v) {
            if (v.size() >= 2 && (v.front() == '"' || v.front() == '\'') && v.back() == v.front()) v = v.substr(1, v.size() - 2);
        };
        unq(l.key);
        unq(l.value);
        out.push_back(l);
    }
    return out;
}

struct KernelInfo {  // Contexts.h:28-51
    string name;
    bool has_barriers = true;
    Dims3 grid{1, 1, 1}, block{1, 1, 1};
    int reg = 32;
    double exec_time = -1;
};
struct FusionInfo {  // Contexts.h:53-62
    string file;
    vector<string> kernels;
};

map<string, KernelInfo> parse_kernels(const string& text, vector<string>* order)
{
    map<string, KernelInfo> out;
    auto ls = yaml_lines(text);
    KernelInfo* cur = nullptr;
    Dims3* dim = nullptr;
    int seen = 0;
    for (auto& l : ls) {
        if (l.indent == 0) {
            if (cur && (seen & 0x1f) != 0x1f) die("kernel '" + cur->name + "': missing required key (KernelName, HasBarriers, GridDim, BlockDim, Reg)");
            if (l.key.empty()) die("kernel config must be a map of name -> KernelInfo");
            cur = &out[l.key];
            cur->name = l.key;
            if (order) order->push_back(l.key);
            seen = 0;
            dim = nullptr;
            continue;
        }
        if (!cur) die("kernel config: entry before any kernel name");
        if (l.key == "KernelName") { cur->name = l.value; seen |= 1; dim = nullptr; }
        else if (l.key == "HasBarriers") { cur->has_barriers = (l.value == "true" || l.value == "True"); seen |= 2; dim = nullptr; }
        else if (l.key == "GridDim") { dim = &cur->grid; seen |= 4; }
        else if (l.key == "BlockDim") { dim = &cur->block; seen |= 8; }
        else if (l.key == "Reg") { cur->reg = atoi(l.value.c_str()); seen |= 16; dim = nullptr; }
        else if (l.key == "ExecTime") { cur->exec_time = atof(l.value.c_str()); dim = nullptr; }
        else if ((l.key == "X" || l.key == "Y" || l.key == "Z") && dim) {
            int v = atoi(l.value.c_str());
            if (v < 1) die("kernel '" + cur->name + "': dimensions must be positive");
            (l.key == "X" ? dim->x : l.key == "Y" ? dim->y : dim->z) = v;
        }
    }
    if (cur && (seen & 0x1f) != 0x1f) die("kernel '" + cur->name + "': missing required key (KernelName, HasBarriers, GridDim, BlockDim, Reg)");
    return out;
}

vector<FusionInfo> parse_fusions(const string& text)
{
    vector<FusionInfo> out;
    bool in_kernels = false;
    for (auto& l : yaml_lines(text)) {
        if (l.dash && l.key == "File") {
            out.push_back({});
            out.back().file = l.value;
            in_kernels = false;
        } else if (l.key == "File" && !out.empty()) {
            out.back().file = l.value;
        } else if (l.key == "Kernels") {
            if (l.dash) out.push_back({});
            if (out.empty()) die("fusion config: Kernels before File");
            in_kernels = true;
        } else if (l.dash && l.key.empty() && in_kernels && !out.empty()) {
            out.back().kernels.push_back(l.value);
        }
    }
    for (auto& f : out)
        if (f.file.empty() || f.kernels.empty()) die("fusion entry needs File and Kernels");
    return out;
}

string dump_kernel_yaml(const map<string, KernelInfo>& ks)
{
    // the layout llvm::yaml::Output gives the reference's {b,h}fuse_kernels.yaml
    stringstream o;
    o << "---\n";
    auto pad = [](const string& k) { return k + ":" + string(k.size() < 16 ? 16 - k.size() : 1, ' '); };
    for (auto& [name, k] : ks) {
        o << name << ":\n";
        o << "  " << pad("KernelName") << k.name << "\n";
        o << "  " << pad("HasBarriers") << (k.has_barriers ? "true" : "false") << "\n";
        o << "  GridDim:\n";
        o << "    " << pad("X") << k.grid.x << "\n    " << pad("Y") << k.grid.y << "\n    " << pad("Z") << k.grid.z << "\n";
        o << "  BlockDim:\n";
        o << "    " << pad("X") << k.block.x << "\n    " << pad("Y") << k.block.y << "\n    " << pad("Z") << k.block.z << "\n";
        o << "  " << pad("Reg") << k.reg << "\n";
    }
    o << "...\n";
    return o.str();
}

// ---- kernel source handling ---------------------------------------------------------------
bool ident_char(char c) { return isalnum((unsigned char)c) || c == '_'; }

// positions of comments and string literals are skipped by every scanner below
size_t skip_trivia(const string& s, size_t i)
{
    if (s.compare(i, 2, "//") == 0) {
        size_t e = s.find('\n', i);
        return e == string::npos ? s.size() : e;
    }
    if (s.compare(i, 2, "/*") == 0) {
        size_t e = s.find("*/", i + 2);
        return e == string::npos ? s.size() : e + 2;
    }
    if (s[i] == '"') {
        size_t e = i + 1;
        while (e < s.size() && s[e] != '"') e += (s[e] == '\\') ? 2 : 1;
        return e + 1;
    }
    return i;
}

size_t match_close(const string& s, size_t open, char oc, char cc)
{
    int depth = 0;
    for (size_t i = open; i < s.size(); ++i) {
        size_t j = skip_trivia(s, i);
        if (j != i) { i = j - 1; continue; }
        if (s[i] == oc) ++depth;
        else if (s[i] == cc && --depth == 0) return i;
    }
    die("unbalanced brackets in kernel source");
}

struct Param {
    string decl_prefix;  // type part, e.g. "float* __restrict__ "
    string name;
};
struct SharedDecl {
    string type, name, extent;  // float A_shared[512]  -> "float", "A_shared", "[512]"
};
struct Kernel {
    string name;
    vector<Param> params;
    string body;  // text between the outer braces
    vector<SharedDecl> shared;
};

// replace whole-identifier occurrences outside comments/strings; `not_after_dot` keeps member names
string replace_ident(const string& s, const string& from, const string& to, bool not_after_dot = true)
{
    string out;
    for (size_t i = 0; i < s.size();) {
        size_t j = skip_trivia(s, i);
        if (j != i) { out.append(s, i, j - i); i = j; continue; }
        if (ident_char(s[i]) && (i == 0 || !ident_char(s[i - 1]))) {
            size_t e = i;
            while (e < s.size() && ident_char(s[e])) ++e;
            const bool member = not_after_dot && i > 0 && (s[i - 1] == '.' || (i > 1 && s[i - 1] == '>' && s[i - 2] == '-'));
            if (!member && s.compare(i, e - i, from) == 0) out += to;
            else out.append(s, i, e - i);
            i = e;
        } else {
            out += s[i++];
        }
    }
    return out;
}

// blockIdx.x -> blockIdx_x_ etc. (whitespace around the dot tolerated)
string rewrite_builtins(const string& s)
{
    static const char* bases[] = {"gridDim", "blockIdx", "blockDim", "threadIdx"};
    string out;
    for (size_t i = 0; i < s.size();) {
        size_t j = skip_trivia(s, i);
        if (j != i) { out.append(s, i, j - i); i = j; continue; }
        bool done = false;
        if (ident_char(s[i]) && (i == 0 || (!ident_char(s[i - 1]) && s[i - 1] != '.'))) {
            for (const char* b : bases) {
                const size_t n = strlen(b);
                if (s.compare(i, n, b) == 0 && (i + n >= s.size() || !ident_char(s[i + n]))) {
                    size_t p = i + n;
                    while (p < s.size() && isspace((unsigned char)s[p])) ++p;
                    if (p < s.size() && s[p] == '.') {
                        ++p;
                        while (p < s.size() && isspace((unsigned char)s[p])) ++p;
                        if (p < s.size() && (s[p] == 'x' || s[p] == 'y' || s[p] == 'z') && (p + 1 >= s.size() || !ident_char(s[p + 1]))) {
                            out += string(b) + "_" + s[p] + "_";
                            i = p + 1;
                            done = true;
                        }
                    }
                    break;
                }
            }
        }
        if (!done) {
            if (ident_char(s[i])) {
                size_t e = i;
                while (e < s.size() && ident_char(s[e])) ++e;
                out.append(s, i, e - i);
                i = e;
            } else {
                out += s[i++];
            }
        }
    }
    return out;
}

Kernel extract_kernel(const string& src, const string& name)
{
    // find `name (` preceded (somewhere before, in the same declaration) by __global__
    for (size_t pos = 0; (pos = src.find(name, pos)) != string::npos; pos += name.size()) {
        if ((pos > 0 && ident_char(src[pos - 1])) || (pos + name.size() < src.size() && ident_char(src[pos + name.size()]))) continue;
        size_t p = pos + name.size();
        while (p < src.size() && isspace((unsigned char)src[p])) ++p;
        if (p >= src.size() || src[p] != '(') continue;
        size_t decl_start = src.find_last_of(";}", pos);
        decl_start = decl_start == string::npos ? 0 : decl_start + 1;
        if (src.substr(decl_start, pos - decl_start).find("__global__") == string::npos) continue;
        const size_t pclose = match_close(src, p, '(', ')');
        size_t b = pclose + 1;
        while (b < src.size() && isspace((unsigned char)src[b])) ++b;
        if (b >= src.size() || src[b] != '{') continue;  // a prototype, not the definition
        const size_t bclose = match_close(src, b, '{', '}');
        Kernel k;
        k.name = name;
        k.body = src.substr(b + 1, bclose - b - 1);
        // parameters: split on top-level commas, name = last identifier
        string plist = src.substr(p + 1, pclose - p - 1);
        int depth = 0;
        string cur;
        vector<string> parts;
        for (char c : plist) {
            if (c == '(' || c == '[' || c == '<') ++depth;
            if (c == ')' || c == ']' || c == '>') --depth;
            if (c == ',' && depth == 0) { parts.push_back(cur); cur.clear(); }
            else cur += c;
        }
        if (!trim(cur).empty()) parts.push_back(cur);
        for (auto& part : parts) {
            string t = trim(part);
            size_t e = t.size();
            while (e > 0 && !ident_char(t[e - 1])) --e;
            size_t s0 = e;
            while (s0 > 0 && ident_char(t[s0 - 1])) --s0;
            if (s0 == e) die("cannot parse parameter '" + t + "' of " + name);
            k.params.push_back({t.substr(0, s0), t.substr(s0, e - s0)});
        }
        return k;
    }
    die("kernel '" + name + "' not found (need a __global__ definition)");
}

// pull `__shared__ T name[N]...;` declarations out of the body (Matchers.cc:322-412)
void hoist_shared(Kernel& k)
{
    string out;
    const string& s = k.body;
    for (size_t i = 0; i < s.size();) {
        size_t j = skip_trivia(s, i);
        if (j != i) { out.append(s, i, j - i); i = j; continue; }
        if (s.compare(i, 10, "__shared__") == 0 && (i == 0 || !ident_char(s[i - 1])) && !ident_char(s[i + 10])) {
            size_t semi = s.find(';', i);
            if (semi == string::npos) die("unterminated __shared__ declaration in " + k.name);
            string decl = trim(s.substr(i + 10, semi - i - 10));
            if (decl.find('=') != string::npos) die("initialised __shared__ declaration in " + k.name);
            size_t br = decl.find('[');
            string head = trim(br == string::npos ? decl : decl.substr(0, br));
            string extent = br == string::npos ? "" : trim(decl.substr(br));
            size_t e = head.size(), s0 = e;
            while (s0 > 0 && ident_char(head[s0 - 1])) --s0;
            SharedDecl d{trim(head.substr(0, s0)), head.substr(s0, e - s0), extent};
            if (d.type.empty() || d.name.empty()) die("cannot parse __shared__ declaration '" + decl + "' in " + k.name);
            if (d.type.find("extern") != string::npos) die("extern __shared__ (dynamic LDS) is not supported: " + k.name);
            k.shared.push_back(d);
            // also accept the attribute spelling the reference's pretty-printer produces
            i = semi + 1;
            continue;
        }
        out += s[i++];
    }
    k.body = out;
}

string indent_block(const string& body, const string& pad)
{
    stringstream in(body), out;
    string line;
    bool blank = true;  // hoisted declarations leave empty lines behind: keep at most one, none at the top
    while (getline(in, line)) {
        const bool empty = trim(line).empty();
        if (!(empty && blank)) out << (empty ? "" : pad + line) << "\n";
        blank = empty;
    }
    return out.str();
}

// ---- emission -----------------------------------------------------------------------------
struct Options {
    bool bfuse = false;
    string out_dir = ".", yaml_dir = ".";
    string fusion_cfg, kernel_cfg, cc_dir = ".";
    int pattern = kZigzag, M = 1, N = 1, chunk = 84, pad = kWaveSize;
};

string dims_assign(const KernelInfo& k, const string& ind)
{
    stringstream o;
    o << ind << "gridDim_x_ = " << k.grid.x << ";\n" << ind << "gridDim_y_ = " << k.grid.y << ";\n" << ind << "gridDim_z_ = " << k.grid.z << ";\n";
    o << ind << "blockDim_x_ = " << k.block.x << ";\n" << ind << "blockDim_y_ = " << k.block.y << ";\n" << ind << "blockDim_z_ = " << k.block.z << ";\n";
    return o.str();
}

string emit_bfuse(const vector<Kernel>& ks, const vector<KernelInfo>& infos, const string& fused_name, const Options& opt,
                  KernelInfo* fused_info)
{
    const int n = (int)ks.size();
    LaunchDims dims[kMaxKernels];
    // A side narrower than the fused block is guarded by `threadIdx.x < T`.  Wavefronts with
    // no lane under the guard skip the branch and run to the end of the kernel, which removes
    // them from the hardware barrier's count; a partly covered wavefront enters the branch and
    // takes part in the barrier as a whole, so T need not be a multiple of 64.
    for (int i = 0; i < n; ++i) dims[i] = {infos[i].grid, infos[i].block};
    const int p0 = opt.pattern == kZigzag ? opt.M : opt.chunk;
    const BlockPlan plan = make_block_plan(opt.pattern, n, dims, p0, opt.N);
    stringstream o;
    o << "#include <hip/hip_runtime.h>\n\n";
    o << "extern \"C\" __global__ __launch_bounds__(" << plan.fused_block << ") void " << fused_name << "(";
    bool first = true;
    for (int i = 0; i < n; ++i)
        for (auto& p : ks[i].params) {
            o << (first ? "" : ", ") << p.decl_prefix << ks[i].name << "_" << p.name << "_";
            first = false;
        }
    o << ")\n{\n  /*\n   * KernelID_ means...\n";
    for (int i = 0; i < n; ++i) o << "   * " << i << ": " << ks[i].name << "\n";
    o << "   */\n";
    o << "  int gridDim_x_, gridDim_y_, gridDim_z_;\n  int blockIdx_x_, blockIdx_y_, blockIdx_z_;\n"
         "  int blockDim_x_, blockDim_y_, blockDim_z_;\n  int threadIdx_x_, threadIdx_y_, threadIdx_z_;\n"
         "  int NewBlockIdx_;\n  int KernelID_;\n  \n";
    const string B = "(int)blockIdx.x";
    bool first_if = true;
    for (int s = 0; s < plan.n_seg; ++s) {
        const Segment& g = plan.seg[s];
        for (int j = 0; j < g.n_slot; ++j) {
            const Slot& sl = g.slot[j];
            o << (first_if ? "  if (" : "  else if (");
            first_if = false;
            o << "(" << B << " >= " << g.lo << " && " << B << " < " << g.hi << ")";
            if (g.n_slot > 1)
                o << " && ((" << B << " - " << g.lo << ") % " << g.period << " >= " << sl.off << ") && ((" << B << " - " << g.lo << ") % "
                  << g.period << " < " << sl.off + sl.width << ")";
            o << ")\n  {\n";
            o << "    NewBlockIdx_ = " << sl.base << " + int((" << B << " - " << g.lo << ") / " << g.period << ") * " << sl.width << " + (("
              << B << " - " << g.lo << ") % " << g.period << " - " << sl.off << ");\n";
            o << "    KernelID_  = " << sl.kern << ";\n" << dims_assign(infos[sl.kern], "    ") << "  }\n";
        }
    }
    o << "  else\n  {\n    return;\n  }\n";
    o << "  blockIdx_x_ = NewBlockIdx_ % gridDim_x_;\n  blockIdx_y_ = NewBlockIdx_ / gridDim_x_ % gridDim_y_;\n"
         "  blockIdx_z_ = NewBlockIdx_ / (gridDim_x_ * gridDim_y_);\n  threadIdx_x_ = (int)threadIdx.x % blockDim_x_;\n"
         "  threadIdx_y_ = (int)threadIdx.x / blockDim_x_ % blockDim_y_;\n  threadIdx_z_ = (int)threadIdx.x / (blockDim_x_ * blockDim_y_);\n\n";
    // union of the sides' static LDS (Tools.cc:219-251)
    bool any_shared = false;
    for (auto& k : ks) any_shared |= !k.shared.empty();
    if (any_shared) {
        for (auto& k : ks) {
            if (k.shared.empty()) continue;
            o << "  typedef struct " << k.name << " {\n";
            for (auto& d : k.shared) o << "     " << d.type << " " << d.name << d.extent << ";\n";
            o << "  } " << k.name << "Ty_;\n";
        }
        o << "  typedef union ShrdUnion {\n";
        for (auto& k : ks)
            if (!k.shared.empty()) o << "    " << k.name << "Ty_ " << k.name << ";\n";
        o << "  } ShrdUnionTy_;\n\n  __shared__ ShrdUnionTy_ SU_;\n\n";
    }
    for (int i = 0; i < n; ++i) {
        string body = ks[i].body;
        for (auto& d : ks[i].shared) body = replace_ident(body, d.name, "SU_." + ks[i].name + "." + d.name);
        o << "  // " << ks[i].name << "\n";
        o << (i == 0 ? "  if " : "  else if ") << "((KernelID_ == " << i << ") && ((int)threadIdx.x < " << infos[i].block.size() << "))\n  {\n";
        o << indent_block(body, "    ") << "  }\n";
    }
    o << "}\n";
    fused_info->grid = {plan.fused_grid, 1, 1};
    fused_info->block = {plan.fused_block, 1, 1};
    return o.str();
}

const char* kSideBarrier = R"(// Barrier over the wavefronts of ONE side of a horizontally fused workgroup (gfx950 has no
// partial-workgroup barrier): lane 0 of every wavefront of the side adds 1 to an LDS counter,
// then the wavefront polls until the counter reaches waves * epoch.  The poll is bounded so
// that the grid always drains; a wait that gives up is counted in bfuse_sync_timeouts, which the
// loader reads after the launch (a side that carried on unsynchronised has a wrong output).
#ifndef BFUSE_SIDE_BARRIER_DEFINED
#define BFUSE_SIDE_BARRIER_DEFINED
extern "C" __device__ unsigned int bfuse_sync_timeouts = 0u;
__device__ __forceinline__ void bfuse_side_barrier(unsigned int* counter, unsigned int waves, unsigned int* epoch)
{
  *epoch += 1u;
  const unsigned int target = waves * (*epoch);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  if ((threadIdx.x & 63) == 0) atomicAdd(counter, 1u);
  unsigned int spins = 0;
  while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < target) {
    __builtin_amdgcn_s_sleep(1);
    if (++spins == (1u << 22)) {
      if ((threadIdx.x & 63) == 0) atomicAdd(&bfuse_sync_timeouts, 1u);
      break;
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}
#endif

)";

string emit_hfuse(const vector<Kernel>& ks, const vector<KernelInfo>& infos, const string& fused_name, const Options& opt,
                  KernelInfo* fused_info)
{
    const int n = (int)ks.size();
    LaunchDims dims[kMaxKernels];
    for (int i = 0; i < n; ++i) dims[i] = {infos[i].grid, infos[i].block};
    const ThreadPlan plan = plan_threads(n, dims, opt.pad);
    // With thread ranges that are not whole wavefronts, lane 0 of a side's wavefront can belong to
    // the other side, and every side barrier would give up.  Such a kernel is still written (its
    // text and launch shape are what the reference's 32-thread padding produces, for comparison),
    // but it refuses to compile.
    bool any_barrier = false;
    for (int i = 0; i < n; ++i) any_barrier = any_barrier || ks[i].body.find("__syncthreads") != string::npos;
    const bool unsafe = opt.pad % kWaveSize != 0 && any_barrier;
    if (opt.pad % kWaveSize != 0)
        cerr << "horizontal-fuser: warning: -w " << opt.pad << " lets one wavefront hold threads of two kernels"
             << (unsafe ? "; " + fused_name + " synchronises, so its output is marked not to be compiled for gfx950\n" : "\n");
    stringstream o;
    o << "#include <hip/hip_runtime.h>\n\n";
    if (unsafe)
        o << "#error \"" << fused_name << ": thread ranges padded to " << opt.pad
          << " are not whole 64-lane wavefronts; the per-side barrier needs -w 64 (or a multiple)\"\n\n";
    o << kSideBarrier;
    o << "extern \"C\" __global__ __launch_bounds__(" << plan.fused_block << ") void " << fused_name << "(";
    bool first = true;
    for (int i = 0; i < n; ++i)
        for (auto& p : ks[i].params) {
            o << (first ? "" : ", ") << p.decl_prefix << ks[i].name << "_" << p.name << "_";
            first = false;
        }
    o << ")\n{\n";
    o << "  __shared__ unsigned int bfuse_arrive_[" << n << "];\n";
    o << "  if ((int)threadIdx.x < " << n << ") bfuse_arrive_[(int)threadIdx.x] = 0u;\n  __syncthreads();\n";
    const string T = "(int)threadIdx.x", B = "(int)blockIdx.x";
    for (int i = 0; i < n; ++i) {
        const KernelInfo& ki = infos[i];
        string body = ks[i].body;
        const unsigned waves = (unsigned)(round_up(ki.block.size(), kWaveSize) / kWaveSize);
        body = replace_ident(body, "__syncthreads", "BFUSE_SIDE_SYNC_");
        // BFUSE_SIDE_SYNC_() -> call with this side's counter
        {
            string t;
            const string from = "BFUSE_SIDE_SYNC_";
            for (size_t p = 0; p < body.size();) {
                if (body.compare(p, from.size(), from) == 0) {
                    size_t q = p + from.size();
                    while (q < body.size() && isspace((unsigned char)body[q])) ++q;
                    if (q < body.size() && body[q] == '(') {
                        size_t c = match_close(body, q, '(', ')');
                        t += "bfuse_side_barrier(&bfuse_arrive_[" + to_string(i) + "], " + to_string(waves) + "u, &bfuse_epoch_)";
                        p = c + 1;
                        continue;
                    }
                }
                t += body[p++];
            }
            body = t;
        }
        o << "  // " << ks[i].name << "\n";
        o << "  if ((" << T << " >= " << plan.thr_lo[i] << " && " << T << " < " << plan.thr_hi[i] << ") && (" << B << " >= 0 && " << B << " < "
          << plan.blocks[i] << "))\n  {\n";
        const string NT = "(" + T + " - " + to_string(plan.thr_lo[i]) + ")";
        o << "      int blockIdx_x_ = " << B << " % " << ki.grid.x << ";\n";
        o << "      int blockIdx_y_ = " << B << " / " << ki.grid.x << " % " << ki.grid.y << ";\n";
        o << "      int blockIdx_z_ = " << B << " / " << ki.grid.x * ki.grid.y << ";\n";
        o << "      int threadIdx_x_ = " << NT << " % " << ki.block.x << ";\n";
        o << "      int threadIdx_y_ = " << NT << " / " << ki.block.x << " % " << ki.block.y << ";\n";
        o << "      int threadIdx_z_ = " << NT << " / " << ki.block.x * ki.block.y << ";\n";
        o << "      int gridDim_x_ = " << ki.grid.x << ", gridDim_y_ = " << ki.grid.y << ", gridDim_z_ = " << ki.grid.z << ";\n";
        o << "      int blockDim_x_ = " << ki.block.x << ", blockDim_y_ = " << ki.block.y << ", blockDim_z_ = " << ki.block.z << ";\n";
        o << "      (void)blockIdx_x_; (void)blockIdx_y_; (void)blockIdx_z_; (void)threadIdx_x_; (void)threadIdx_y_; (void)threadIdx_z_;\n";
        o << "      (void)gridDim_x_; (void)gridDim_y_; (void)gridDim_z_; (void)blockDim_x_; (void)blockDim_y_; (void)blockDim_z_;\n";
        o << "      unsigned int bfuse_epoch_ = 0u; (void)bfuse_epoch_;\n";
        o << indent_block(body, "    ") << "  }\n";
    }
    o << "}\n";
    fused_info->grid = {plan.fused_grid, 1, 1};
    fused_info->block = {plan.fused_block, 1, 1};
    return o.str();
}

void print_help(const char* prog)
{
    cout << "Usage: " << prog << " [-h] [-b] [-y yaml_output] [-o output] [-p pattern] [-M m] [-N n] [-c chunk] [-w pad] fusion_config kernel_config compile_commands\n";
    cout << "Options:\n";
    cout << " -h                : Print this page.\n";
    cout << " -b                : Process Block-level fusion.                   (default: false)\n";
    cout << " -y                : Write output yaml to the directory.           (default: .)\n";
    cout << " -o                : Write output file to the directory.           (default: .)\n";
    cout << " -p                : Block pattern: zigzag, proportional, chunked, ranges. (default: zigzag)\n";
    cout << " -M, -N            : zig-zag ratio cap and multiplier.             (default: 1, 1)\n";
    cout << " -c                : chunk size (chunked) / min-option (proportional). (default: 84)\n";
    cout << " -w                : thread-range padding of horizontal fusion.    (default: 64)\n";
    cout << "\n";
    cout << "fusion_config      : YAML file about fusion configuration.\n";
    cout << "kernel_config      : YAML file about kernel configuration.\n";
    cout << "compile_commands   : the directory where the kernel source (and 'compile_commands.json') is located.\n";
}

}  // namespace

int main(int argc, char** argv)
{
    if (argc < 3) {
        print_help(argv[0]);
        return 0;
    }
    Options opt;
    int c;
    while ((c = getopt(argc, argv, "hbo:y:p:M:N:c:w:")) != -1) {
        switch (c) {
            case 'o': opt.out_dir = optarg; break;
            case 'y': opt.yaml_dir = optarg; break;
            case 'b': opt.bfuse = true; break;
            case 'p': {
                string p = optarg;
                if (p == "zigzag") opt.pattern = kZigzag;
                else if (p == "proportional") opt.pattern = kProportional;
                else if (p == "chunked") opt.pattern = kChunked;
                else if (p == "ranges") opt.pattern = kRanges;
                else die("unknown pattern '" + p + "'");
                break;
            }
            case 'M': opt.M = atoi(optarg); break;
            case 'N': opt.N = atoi(optarg); break;
            case 'c': opt.chunk = atoi(optarg); break;
            case 'w': opt.pad = atoi(optarg); break;
            case 'h':
            default: print_help(argv[0]); return 0;
        }
    }
    if (argc - optind < 2) {
        print_help(argv[0]);
        return 0;
    }
    opt.fusion_cfg = argv[optind];
    opt.kernel_cfg = argv[optind + 1];
    if (argc - optind > 2) opt.cc_dir = argv[optind + 2];
    if (opt.M < 1 || opt.N < 1 || opt.chunk < 1 || opt.pad < 1) die("-M, -N, -c and -w must be positive");
    cout << "fusion config: " << opt.fusion_cfg << "\n";
    cout << "kernel config: " << opt.kernel_cfg << "\n";
    cout << "compile commands: " << opt.cc_dir << "\n";

    const auto fusions = parse_fusions(read_file(opt.fusion_cfg));
    const auto kernels = parse_kernels(read_file(opt.kernel_cfg), nullptr);
    map<string, KernelInfo> fused_yaml;
    map<string, string> unfused;  // the input kernels, re-declared in the attribute order HIP accepts
    for (size_t f = 0; f < fusions.size(); ++f) {
        const FusionInfo& fi = fusions[f];
        if ((int)fi.kernels.size() > kMaxKernels) die("at most " + to_string(kMaxKernels) + " kernels per fusion");
        const string src = read_file(opt.cc_dir + "/" + fi.file);
        vector<Kernel> ks;
        vector<KernelInfo> infos;
        string fused_name, file_name;
        for (auto& kn : fi.kernels) {
            auto it = kernels.find(kn);
            if (it == kernels.end()) die("kernel '" + kn + "' is not in " + opt.kernel_cfg);  // map::at in the reference (Contexts.cc:69)
            infos.push_back(it->second);
            Kernel k = extract_kernel(src, kn);
            if (!unfused.count(kn)) {
                // CUDA lets `__launch_bounds__` follow the return type (TVM prints it there); hipcc does not
                const KernelInfo& ki = it->second;
                stringstream u;
                u << "extern \"C\" __global__ __launch_bounds__(" << ki.block.x * ki.block.y * ki.block.z << ") void " << kn << "(";
                for (size_t a = 0; a < k.params.size(); ++a) u << (a ? ", " : "") << k.params[a].decl_prefix << k.params[a].name;
                u << ")\n{" << k.body << "}\n";
                unfused[kn] = u.str();
            }
            // block fusion overlays the LDS arrays of the sides in one union; thread fusion leaves
            // every `__shared__` declaration where it is, so the sides' LDS adds up (Matchers.cc:322-412)
            if (opt.bfuse) hoist_shared(k);
            for (auto& p : k.params) k.body = replace_ident(k.body, p.name, kn + "_" + p.name + "_");
            k.body = rewrite_builtins(k.body);
            ks.push_back(k);
            fused_name += kn + "_";
            file_name += kn + "_";
        }
        fused_name += opt.bfuse ? "fused_bfuse" : "fused_hfuse";
        file_name += opt.bfuse ? "bfuse.hip" : "hfuse.hip";
        cout << "(" << f + 1 << "/" << fusions.size() << ") Start to " << (opt.bfuse ? "bfuse" : "hfuse") << " \"" << fused_name << "\" kernel...\n";
        KernelInfo fused;
        fused.name = fused_name;
        fused.has_barriers = true;  // as the reference records them (Fuse.cc:204-209)
        fused.reg = 32;
        const string text = opt.bfuse ? emit_bfuse(ks, infos, fused_name, opt, &fused) : emit_hfuse(ks, infos, fused_name, opt, &fused);
        write_file(opt.out_dir, file_name, text);
        fused_yaml[fused_name] = fused;
    }
    write_file(opt.yaml_dir, opt.bfuse ? "bfuse_kernels.yaml" : "hfuse_kernels.yaml", dump_kernel_yaml(fused_yaml));
    string all = "#include <hip/hip_runtime.h>\n\n";
    for (auto& kv : unfused) all += kv.second + "\n";
    write_file(opt.out_dir, "kernels.hip", all);
    return 0;
}
