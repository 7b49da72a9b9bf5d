// Stored graph format: <dir>/graph.dr (text) + <dir>/N.var (raw little-endian fp32), byte compatible
// with the reference's writer and reader (src/dR_parser.c:58-180 and :182-523).
//
//   deepRACIN graph: <N> nodes, <F> feed nodes
//   Node <id>: <Desc>
//   params: p0 p1 ...
//   previous_nodes: i j ...
//   next_nodes: ...            (written for humans, ignored when reading)
//   variable_files: a.var b.var
//
// Reader rules kept from the reference: lines are split on any run of '\r' / '\n', fields on runs
// of ' '; the node count is the 3rd and the feed count the 5th token of the header; node ids index
// the returned node list; the description is matched by prefix.
#include "dr_internal.hpp"

#include <sys/stat.h>
#include <cerrno>

using namespace dr;

namespace {

std::vector<std::string> split(const std::string& s, const char* delims) {
    std::vector<std::string> out;
    size_t i = 0;
    while (i < s.size()) {
        size_t b = s.find_first_not_of(delims, i);
        if (b == std::string::npos) break;
        size_t e = s.find_first_of(delims, b);
        if (e == std::string::npos) e = s.size();
        out.push_back(s.substr(b, e - b));
        i = e;
    }
    return out;
}

bool read_file(const std::string& path, std::string* out) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) return false;
    fseek(f, 0, SEEK_END);
    long n = ftell(f);
    fseek(f, 0, SEEK_SET);
    out->resize(n > 0 ? (size_t)n : 0);
    size_t got = n > 0 ? fread(&(*out)[0], 1, (size_t)n, f) : 0;
    fclose(f);
    return got == (size_t)(n > 0 ? n : 0);
}

std::string join_path(const std::string& a, const std::string& b) {
    if (a.empty()) return b;
    return a[a.size() - 1] == '/' ? a + b : a + "/" + b;
}

bool mkdir_p(const std::string& path) {
    std::string cur;
    for (size_t i = 0; i <= path.size(); ++i) {
        if (i == path.size() || path[i] == '/') {
            if (!cur.empty() && mkdir(cur.c_str(), 0777) != 0 && errno != EEXIST) return false;
        }
        if (i < path.size()) cur += path[i];
    }
    struct stat st;
    return stat(path.c_str(), &st) == 0 && S_ISDIR(st.st_mode);
}

typedef dR_Node* (*Factory)(dR_Graph*, dR_Node**, gint, gchar**, gint, gfloat**, gint);
struct Kind { const char* prefix; Factory make; int minInputs, maxInputs; };

// Prefix order matters (the reference tests "Conv2D" before anything else, src/dR_parser.c:336).
const Kind kKinds[] = {
    { "Conv2D",         dR_conv2d_parseAppendNode,       1, 1 },
    { "Pooling",        dR_pooling_parseAppendNode,      1, 1 },
    { "FullyConnected", dR_fc_parseAppendNode,           1, 1 },
    { "Softmax",        dR_softmax_parseAppendNode,      1, 1 },
    { "Slice",          dR_slice_parseAppendNode,        1, 1 },
    { "Concat",         dR_concat_parseAppendNode,       2, 256 },
    { "ElemWise1Op",    dR_elemwise1op_parseAppendNode,  1, 1 },
    { "Normalization",  dR_norm_parseAppendNode,         1, 1 },
    { "DataFeedNode",   dR_datafeednode_parseAppendNode, 0, 0 },
};

// Node kinds of the reference that exist in graph.dr files but lie outside the CNN layer path.
const char* const kForeign[] = { "PPFilter", "MaskDependentFilter", "LabelCreation", "Upscaling",
                                 "RGB2Gray", "ResolveRoI", "CropOrPad", "ElemWise2Op" };

}  // namespace

extern "C" {

gboolean dR_serializeGraph(dR_Graph* net, gchar* path) {
    const std::string folder = join_path(path ? path : "", "dr_graph_export");
    if (!mkdir_p(folder)) {
        say("Error: Could not create folder %s.\n", folder.c_str());
        return FALSE;
    }
    char header[96];
    snprintf(header, sizeof header, "deepRACIN graph: %d nodes, %d feed nodes", net->allNodes->length, net->feed_layers->length);
    std::string text = header;
    int varCounter = 0;
    for (dR_Node* node : nodes_of(net->allNodes)) {
        gchar* params[10];
        gfloat* variables[2];
        gint sizes[2], numParams = 10, numVars = 2;
        gchar* desc = node->serializeNode(node, params, &numParams, variables, sizes, &numVars);
        if (!desc) { say("Error: node %d could not be serialized.\n", node->layerID); return FALSE; }
        char head[128];
        snprintf(head, sizeof head, "\nNode %d: %s\nparams:", node->layerID, desc);
        text += head;
        for (int i = 0; i < numParams; ++i) { text += " "; text += params[i]; free(params[i]); }
        text += "\nprevious_nodes:";
        for (dR_Node* p : nodes_of(node->previous_layers)) text += " " + std::to_string(p->layerID);
        text += "\nnext_nodes:";
        for (dR_Node* p : nodes_of(node->next_layers)) text += " " + std::to_string(p->layerID);
        text += "\nvariable_files:";
        for (int i = 0; i < numVars; ++i) {
            const std::string name = std::to_string(varCounter++) + ".var";
            text += " " + name;
            FILE* f = fopen(join_path(folder, name).c_str(), "wb");
            if (!f) { say("Error while creating the variable file %s.\n", name.c_str()); return FALSE; }
            const size_t wrote = fwrite(variables[i], sizeof(float), (size_t)sizes[i], f);
            fclose(f);
            if (wrote != (size_t)sizes[i]) { say("Error while writing the variable file %s.\n", name.c_str()); return FALSE; }
        }
    }
    text += "\n";
    FILE* f = fopen(join_path(folder, "graph.dr").c_str(), "wb");
    if (!f) { say("Error while creating graph.dr in %s.\n", folder.c_str()); return FALSE; }
    fwrite(text.data(), 1, text.size(), f);
    fclose(f);
    return TRUE;
}

dR_Node* dR_parseGraph(dR_Graph* net, gchar* path, dR_Node*** outnodes, gint* numnodes, dR_Node*** outfeednodes,
                       gint* numfeednodes) {
    if (net->number_of_layers != 0) {
        say("dR_parseGraph can only fill an empty graph! Given graph not empty!\n");
        return NULL;
    }
    const std::string dir = path ? path : "";
    net->config->modelPath = strdup(dir.c_str());
    if (verbose(net)) say("Loading Model File %s ...\n", dir.c_str());

    std::string content;
    if (!read_file(join_path(dir, "graph.dr"), &content)) {
        say("Error while opening the graph file.\n");
        return NULL;
    }
    const std::vector<std::string> lines = split(content, "\r\n");
    if (lines.empty()) { say("Parsing Error: graph file is empty.\n"); return NULL; }
    const std::vector<std::string> head = split(lines[0], " ");
    if (head.size() < 5) { say("Parsing Error: malformed header line.\n"); return NULL; }
    const int N = atoi(head[2].c_str()), F = atoi(head[4].c_str());
    if (N <= 0 || F < 0 || F > N || lines.size() < 1 + 5 * (size_t)N) {
        say("Parsing Error: header announces %d nodes and %d feed nodes but the file holds %zu lines.\n", N, F, lines.size());
        return NULL;
    }
    if (verbose(net)) say("Found graph with %d nodes and %d feed nodes.\n", N, F);

    dR_Node** nodes = (dR_Node**)calloc((size_t)N, sizeof(dR_Node*));
    dR_Node** feeds = (dR_Node**)calloc((size_t)(F > 0 ? F : 1), sizeof(dR_Node*));
    int feedCount = 0;
    auto fail_out = [&]() -> dR_Node* { free(nodes); free(feeds); return NULL; };

    for (int i = 0; i < N; ++i) {
        const std::vector<std::string> l0 = split(lines[1 + 5 * i + 0], " ");
        std::vector<std::string> pars = split(lines[1 + 5 * i + 1], " ");
        std::vector<std::string> prev = split(lines[1 + 5 * i + 2], " ");
        std::vector<std::string> vars = split(lines[1 + 5 * i + 4], " ");
        if (l0.size() < 3 || pars.empty() || prev.empty() || vars.empty()) { say("Parsing Error: malformed record of node %d.\n", i); return fail_out(); }
        const int id = atoi(l0[1].c_str());
        const std::string desc = l0[2];
        pars.erase(pars.begin()); prev.erase(prev.begin()); vars.erase(vars.begin());     // drop the labels
        if (id < 0 || id >= N || nodes[id]) { say("Parsing Error: bad or repeated node id %d.\n", id); return fail_out(); }
        if (pars.size() > 10 || vars.size() > 2 || prev.size() > 256) { say("Parsing Error: node %d has too many fields.\n", id); return fail_out(); }
        if (debug(net)) say("Found %s with id %d, %zu params and %zu variables\n", desc.c_str(), id, pars.size(), vars.size());

        std::vector<dR_Node*> inputs;
        for (const std::string& p : prev) {
            const int pid = atoi(p.c_str());
            if (pid < 0 || pid >= N || !nodes[pid]) { say("Parsing Error: node %d refers to node %d which is not defined before it.\n", id, pid); return fail_out(); }
            inputs.push_back(nodes[pid]);
        }
        std::vector<std::string> blobs(vars.size());
        gfloat* variables[2] = { NULL, NULL };
        parse_var_floats[0] = parse_var_floats[1] = 0;
        for (size_t v = 0; v < vars.size(); ++v) {
            const std::string vp = join_path(dir, vars[v]);
            if (!read_file(vp, &blobs[v]) || blobs[v].size() < sizeof(float)) {
                say("Error while opening variable file: %s\n", vp.c_str());
                parse_var_floats[0] = parse_var_floats[1] = 0;
                return fail_out();
            }
            variables[v] = (gfloat*)&blobs[v][0];
            parse_var_floats[v] = blobs[v].size() / sizeof(float);
        }
        std::vector<gchar*> parv;
        for (std::string& p : pars) parv.push_back(&p[0]);

        const Kind* kind = NULL;
        for (const Kind& k : kKinds)
            if (desc.compare(0, strlen(k.prefix), k.prefix) == 0) { kind = &k; break; }
        dR_Node* node = NULL;
        if (!kind) {
            bool foreign = false;
            for (const char* f : kForeign) foreign = foreign || desc.compare(0, strlen(f), f) == 0;
            if (foreign) say("Parsing Error: node type %s is not part of the CNN layer path this library serves!\n", desc.c_str());
            else say("Parsing Error: Node could not be identified: %s!\n", desc.c_str());
        } else if ((int)inputs.size() < kind->minInputs || (int)inputs.size() > kind->maxInputs) {
            say("Failed to parse %s node!\n", kind->prefix);
        } else {
            node = kind->make(net, inputs.empty() ? NULL : inputs.data(), (gint)inputs.size(), parv.empty() ? NULL : parv.data(),
                              (gint)parv.size(), variables, (gint)vars.size());
            if (!node) say("Parsing Error: Node could not be appended!\n");
        }
        parse_var_floats[0] = parse_var_floats[1] = 0;
        if (!node) return fail_out();
        nodes[id] = node;
        if (node->type == tDataFeedNode) {
            if (feedCount >= F) { say("Parsing Error: more feed nodes than the header announces.\n"); return fail_out(); }
            feeds[feedCount++] = node;
        }
    }
    *outnodes = nodes;
    *outfeednodes = feeds;
    *numnodes = N;
    *numfeednodes = F;
    return nodes[N - 1];
}

void dR_printNet(dR_Graph* net, char* path) {
    std::string text = "deepRACIN graph on HIP/gfx950\n";
    for (dR_Node* n : nodes_of(net->allNodes)) {
        if (!n->printLayer) continue;
        gchar* s = n->printLayer(n);
        if (s) { text += s; free(s); }
        if (n->propagated) {
            char shape[96];
            snprintf(shape, sizeof shape, " Output: %dx%dx%d\n", n->oshape.s0, n->oshape.s1, n->oshape.s2);
            text += shape;
        }
    }
    if (!path) { say("%s", text.c_str()); return; }
    FILE* f = fopen(path, "w");
    if (!f) { say("dR_printNet: cannot write %s\n", path); return; }
    fwrite(text.data(), 1, text.size(), f);
    fclose(f);
}

void dR_printSchedule(dR_Graph* net) {
    if (!net->scheduledLayers) return;
    say("Schedule:");
    for (dR_Node* n : nodes_of(net->scheduledLayers)) say(" %d", n->layerID);
    say("\n");
}

}  // extern "C"
