// HCCL_ALGO: the reference's grammar (src/common/alg_parse.cc:120-437) and what its clauses select here.
#include "algo_config.h"

#include <cctype>
#include <set>

namespace hccl_amd {
namespace {

// The reference's vocabularies (alg_parse.cc:34-86), lower case.
const std::set<std::string>& OpTypes()
{
    static const std::set<std::string> names = {"allgather", "allgatherv", "allreduce", "alltoall", "alltoallv",
                                                "alltoallvc", "barrier", "batchsendrecv", "broadcast", "reduce",
                                                "reducescatter", "reducescatterv", "scatter", "send", "recv"};
    return names;
}

const std::set<std::string>& ExecutorTypes()
{
    static const std::set<std::string> names = {"sole", "sequence", "parallel", "pipeline", "concur", "strictordered"};
    return names;
}

const std::set<std::string>& TemplateTypes()
{
    static const std::set<std::string> names = {
        "mesh", "mesh2die", "meshoneshot", "meshtwoshot", "meshconcur", "meshmultilink", "meshchunk",
        "meshchunktwoshot", "meshchunkconcur", "nhr", "nhrmultilink", "nhraicpureduce", "hdaicpureduce", "hd",
        "meshsinglechannel", "nhrmultijetty", "meshmultijetty", "meshconcurrent", "pairwise", "rhd"};
    return names;
}

std::string Lower(const std::string& s)
{
    std::string r = s;
    for (char& c : r) {
        c = static_cast<char>(std::tolower(static_cast<unsigned char>(c)));
    }
    return r;
}

// mesh_chunk and meshChunk both name "meshchunk" (the reference turns underscores into camel case, then lowers).
std::string TemplateKey(const std::string& name)
{
    std::string r;
    for (char c : name) {
        if (c != '_') {
            r += static_cast<char>(std::tolower(static_cast<unsigned char>(c)));
        }
    }
    return r;
}

class Parser {
public:
    explicit Parser(const std::string& input) : in_(input) {}

    HcclResult Run(std::vector<AlgoSegment>* out)
    {
        SkipBlanks();
        while (!AtEnd()) {
            AlgoSegment seg;
            std::vector<int> levels;
            if (!Segment(&seg, &levels)) {
                return HCCL_E_PARA;
            }
            Compact(&seg, levels);
            out->push_back(std::move(seg));
            SkipBlanks();
            if (Eat(';')) {
                SkipBlanks();
                continue;
            }
            break;
        }
        SkipBlanks();
        return AtEnd() ? HCCL_SUCCESS : HCCL_E_PARA;
    }

private:
    const std::string& in_;
    size_t pos_ = 0;

    char Peek(size_t ahead = 0) const { return pos_ + ahead < in_.size() ? in_[pos_ + ahead] : '\0'; }
    bool AtEnd() const { return pos_ >= in_.size(); }
    bool Eat(char c)
    {
        if (Peek() == c) {
            ++pos_;
            return true;
        }
        return false;
    }
    void SkipBlanks()
    {
        while (!AtEnd() && std::isspace(static_cast<unsigned char>(in_[pos_]))) {
            ++pos_;
        }
    }
    bool Identifier(std::string* name)
    {
        SkipBlanks();
        const size_t start = pos_;
        while (!AtEnd() && (std::isalnum(static_cast<unsigned char>(in_[pos_])) || in_[pos_] == '_' || in_[pos_] == '-')) {
            ++pos_;
        }
        if (pos_ == start) {
            return false;
        }
        *name = in_.substr(start, pos_ - start);
        return true;
    }

    // Templates with an explicit level go to that position, the others to the end of the list as it then is;
    // positions nobody filled disappear (alg_parse.cc:156-190).
    static void Place(AlgoSegment* seg, std::vector<int>* filled, AlgoTemplate t, int level)
    {
        if (level < 0) {
            seg->templates.push_back(std::move(t));
            filled->push_back(1);
            return;
        }
        if (static_cast<size_t>(level) >= seg->templates.size()) {
            seg->templates.resize(level + 1);
            filled->resize(level + 1, 0);
        }
        seg->templates[level] = std::move(t);
        (*filled)[level] = 1;
    }
    static void Compact(AlgoSegment* seg, const std::vector<int>& filled)
    {
        std::vector<AlgoTemplate> kept;
        for (size_t i = 0; i < seg->templates.size(); ++i) {
            if (i < filled.size() && filled[i] && !seg->templates[i].name.empty()) {
                kept.push_back(std::move(seg->templates[i]));
            }
        }
        seg->templates = std::move(kept);
    }

    bool Segment(AlgoSegment* seg, std::vector<int>* filled)
    {
        const size_t save = pos_;
        std::string name;
        if (Identifier(&name)) {
            SkipBlanks();
            if (Peek() == ':' && Peek(1) != ':') {
                Eat(':');
                seg->opType = Lower(name);
                if (OpTypes().count(seg->opType) == 0) {
                    return false;
                }
                SkipBlanks();
            } else {
                pos_ = save;
            }
        }
        return ExecutorExpr(seg, filled);
    }

    bool ExecutorExpr(AlgoSegment* seg, std::vector<int>* filled)
    {
        SkipBlanks();
        const size_t save = pos_;
        std::string name;
        if (Identifier(&name)) {
            SkipBlanks();
            if (Lower(name) == "not" && Peek() == '(') {
                Eat('(');
                SkipBlanks();
                if (!Unit(seg, filled)) {
                    return false;
                }
                SkipBlanks();
                if (!Eat(')')) {
                    return false;
                }
                seg->enable = false;
                return true;
            }
            pos_ = save;
        }
        return Unit(seg, filled);
    }

    bool Unit(AlgoSegment* seg, std::vector<int>* filled)
    {
        SkipBlanks();
        std::string name;
        if (!Identifier(&name)) {
            return false;
        }
        SkipBlanks();
        if (Peek() == '{') {
            seg->executor = Lower(name);
            if (ExecutorTypes().count(seg->executor) == 0) {
                return false;
            }
            Eat('{');
            if (!TemplateList(seg, filled)) {
                return false;
            }
            SkipBlanks();
            return Eat('}');
        }
        AlgoTemplate t;
        t.name = TemplateKey(name);
        if (TemplateTypes().count(t.name) == 0) {
            return false;
        }
        seg->executor = "sole";
        Place(seg, filled, std::move(t), -1);
        return true;
    }

    bool TemplateList(AlgoSegment* seg, std::vector<int>* filled)
    {
        SkipBlanks();
        if (Peek() == '}') {
            return true;
        }
        while (true) {
            AlgoTemplate t;
            int level = -1;
            if (!TemplateItem(&t, &level)) {
                return false;
            }
            Place(seg, filled, std::move(t), level);
            SkipBlanks();
            if (!Eat(',')) {
                return true;
            }
            SkipBlanks();
        }
    }

    bool TemplateItem(AlgoTemplate* t, int* level)
    {
        SkipBlanks();
        const size_t save = pos_;
        std::string name;
        if (Identifier(&name)) {
            if (name.size() > 5 && Lower(name.substr(0, 5)) == "level") {
                bool digits = true;
                for (size_t i = 5; i < name.size(); ++i) {
                    digits = digits && std::isdigit(static_cast<unsigned char>(name[i]));
                }
                if (digits) {
                    SkipBlanks();
                    if (Eat('=')) {
                        if (name.size() > 5 + 3) {
                            return false;   // (the reference takes any level that fits 32 bits; a list that long is a typing error)
                        }
                        *level = std::stoi(name.substr(5));
                        SkipBlanks();
                        return TemplateExpr(t);
                    }
                }
            }
            pos_ = save;
        }
        return TemplateExpr(t);
    }

    bool TemplateExpr(AlgoTemplate* t)
    {
        SkipBlanks();
        const size_t save = pos_;
        std::string name;
        if (Identifier(&name)) {
            SkipBlanks();
            if (Lower(name) == "not" && Peek() == '(') {
                Eat('(');
                SkipBlanks();
                if (!TemplateAtom(t)) {
                    return false;
                }
                t->enable = false;
                SkipBlanks();
                return Eat(')');
            }
            pos_ = save;
        }
        return TemplateAtom(t);
    }

    bool TemplateAtom(AlgoTemplate* t)
    {
        SkipBlanks();
        std::string name;
        if (!Identifier(&name)) {
            return false;
        }
        t->name = TemplateKey(name);
        return TemplateTypes().count(t->name) != 0;
    }
};

bool IsMeshFamily(const std::string& t) { return t.compare(0, 4, "mesh") == 0 || t == "pairwise"; }
bool IsNhrFamily(const std::string& t) { return t.compare(0, 3, "nhr") == 0; }
bool IsRhdFamily(const std::string& t) { return t == "rhd" || t == "hd" || t == "hdaicpureduce"; }

// The fold order between the participants of one level under template `t`, per operator.  The reference's
// registered names this follows: Aicpu<Op>Sole<Template> and Aicpu<Op>Sequence<L0><L1>
// (REGISTER_EXECUTOR_* in src/ops/<op>/algorithm/executor/*.cc).
bool OrderOf(HcclAmdOpKind op, const std::string& t, HcclAmdAlgo* algo)
{
    if (t == "meshchunk" || t == "meshchunktwoshot" || t == "meshchunkconcur") {
        *algo = HCCL_AMD_ALGO_MESH_CHUNK;
        return op != HCCL_AMD_OP_REDUCE;
    }
    if (t == "nhraicpureduce") {
        // host-reduce NHR: AllReduce and Reduce gather and fold in rank order, ReduceScatter folds the own slice first
        *algo = op == HCCL_AMD_OP_ALL_REDUCE ? HCCL_AMD_ALGO_RING : HCCL_AMD_ALGO_MESH;
        return true;
    }
    if (t == "meshconcur" && op == HCCL_AMD_OP_ALL_REDUCE) {
        *algo = HCCL_AMD_ALGO_MESH_CONCUR;   // Aicpu AllReduce Sole MeshConcur: mesh ReduceScatter + AllGather
        return true;
    }
    if (op == HCCL_AMD_OP_REDUCE && IsMeshFamily(t)) {
        *algo = t == "meshtwoshot" ? HCCL_AMD_ALGO_MESH_TWO_SHOT : HCCL_AMD_ALGO_MESH;
        return true;
    }
    if (IsMeshFamily(t)) {
        *algo = HCCL_AMD_ALGO_MESH;
        return true;
    }
    if (IsNhrFamily(t)) {
        *algo = HCCL_AMD_ALGO_NHR;
        return true;
    }
    if (IsRhdFamily(t)) {
        *algo = HCCL_AMD_ALGO_RHD;
        return true;
    }
    return false;
}

bool OpKindOf(const std::string& opType, HcclAmdOpKind* kind)
{
    if (opType == "allreduce") {
        *kind = HCCL_AMD_OP_ALL_REDUCE;
    } else if (opType == "reducescatter" || opType == "reducescatterv") {
        *kind = HCCL_AMD_OP_REDUCE_SCATTER;
    } else if (opType == "reduce") {
        *kind = HCCL_AMD_OP_REDUCE;
    } else {
        return false;
    }
    return true;
}

}  // namespace

HcclResult ParseHcclAlgo(const std::string& config, std::vector<AlgoSegment>* segments)
{
    segments->clear();
    if (config.empty()) {
        return HCCL_SUCCESS;
    }
    Parser p(config);
    HcclResult rc = p.Run(segments);
    if (rc != HCCL_SUCCESS) {
        segments->clear();
    }
    return rc;
}

AlgoSelection SelectFromHcclAlgo(const std::vector<AlgoSegment>& segments)
{
    AlgoSelection sel;
    for (size_t k = segments.size(); k-- > 0;) {
        const AlgoSegment& seg = segments[k];
        if (!seg.enable || seg.templates.empty()) {
            continue;
        }
        bool negated = false;
        for (const AlgoTemplate& t : seg.templates) {
            negated = negated || !t.enable;
        }
        if (negated) {
            continue;
        }
        for (int op = 0; op < HCCL_AMD_OP_COUNT; ++op) {
            const HcclAmdOpKind kind = static_cast<HcclAmdOpKind>(op);
            if (sel.set[op]) {
                continue;
            }
            HcclAmdOpKind named;
            if (!seg.opType.empty() && (!OpKindOf(seg.opType, &named) || named != kind)) {
                continue;
            }
            HcclAmdAlgo algo;
            bool twoLevel = false;
            if (seg.executor == "strictordered") {
                if (kind == HCCL_AMD_OP_REDUCE) {
                    continue;
                }
                algo = HCCL_AMD_ALGO_ORDER_PRESERVED;
            } else if (seg.templates.size() == 1) {
                if (!OrderOf(kind, seg.templates[0].name, &algo)) {
                    continue;
                }
            } else if (kind == HCCL_AMD_OP_REDUCE && seg.executor == "sequence" && seg.templates.size() == 2 &&
                       seg.templates[0].name == "nhraicpureduce" && seg.templates[1].name == "nhr") {
                // Aicpu Reduce Sequence NHRAicpuReduce NHR: a mesh ReduceScatter inside the groups and the host-reduce
                // template between them, whatever the name says (reduce_sequence_executor_aicpu_3level.cc:1010-1013)
                algo = HCCL_AMD_ALGO_MESH;
                twoLevel = true;
            } else if ((seg.templates.size() == 2 || seg.templates.size() == 3) && seg.executor == "sequence" &&
                       IsMeshFamily(seg.templates[0].name) && seg.templates[0].name.compare(0, 9, "meshchunk") != 0) {
                // a mesh inside the level-0 groups (the mesh-chunk templates fold in another order there, which is
                // not built), the second template between them and, with a third level, the same one once more
                // (the reference registers Sequence MeshConcur NHR NHR and ... RHD RHD, no mixed forms)
                if (!OrderOf(kind, seg.templates[1].name, &algo) ||
                    (algo != HCCL_AMD_ALGO_RHD && algo != HCCL_AMD_ALGO_NHR && algo != HCCL_AMD_ALGO_MESH &&
                     algo != HCCL_AMD_ALGO_RING)) {
                    continue;
                }
                if (seg.templates[1].name == "nhraicpureduce") {
                    if (seg.templates.size() == 3) {
                        continue;                // the host-reduce executors know two levels
                    }
                    algo = HCCL_AMD_ALGO_MESH;   // between the groups: the own-first fold of the host-reduce template
                } else if (algo == HCCL_AMD_ALGO_MESH || algo == HCCL_AMD_ALGO_RING) {
                    continue;                    // a mesh between the groups: another executor family
                }
                HcclAmdAlgo third;
                if (seg.templates.size() == 3 && (!OrderOf(kind, seg.templates[2].name, &third) || third != algo ||
                                                  seg.templates[2].name == "nhraicpureduce")) {
                    continue;
                }
                twoLevel = true;
            } else {
                continue;   // the other executors over several levels (parallel, pipeline, concur) are not built
            }
            sel.set[op] = true;
            sel.algo[op] = algo;
            sel.twoLevel[op] = twoLevel;
        }
    }
    return sel;
}

}  // namespace hccl_amd
