// ifa_trace_run -- replays a trace of token-id steps through the InferenceEngine and writes the logits it asks for.
//
//   ifa_trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N
//
// DIR holds config.json (with a registered "architecture") and model.safetensors.  Steps come on standard input, one JSON object per
// line: {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}.  A new id starts a query with its
// tokens (AddQuery); a known id continues its query with the given tokens (CommitInferenceResult: the next tokens are the trace's,
// nothing is sampled); one Infer() runs the step for every query at once; "end" removes queries (their slots are free again).
// The fp32 logits of the wanted token places go to <out>/<step>.f32 in the order of the entries ([wanted][vocab], little-endian);
// after every step a line "done <step>" is printed and flushed.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <map>
#include <string>

#include "inference_engine.h"
#include "ifa_json.h"

using namespace inferflow_amd;

int main(int argc, char **argv)
{
    std::string model, dtype = "bfloat16", out;
    int max_tokens = 4096, max_queries = 1024;
    for (int i = 1; i < argc; i++) {
        const std::string a = argv[i];
        auto next = [&]() -> const char * { return i + 1 < argc ? argv[++i] : ""; };
        if (a == "--model") model = next();
        else if (a == "--dtype") dtype = next();
        else if (a == "--out") out = next();
        else if (a == "--max-tokens") max_tokens = atoi(next());
        else if (a == "--max-queries") max_queries = atoi(next());
        else { fprintf(stderr, "unknown option %s\n", a.c_str()); return 2; }
    }
    if (model.empty() || out.empty() || max_tokens < 1) { fprintf(stderr, "usage: %s --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N\n", argv[0]); return 2; }
    InferenceConfig cfg;
    // a query holds at most max_tokens tokens (AddQuery wants room for one more)
    if (!InferenceEngine::LoadConfigForModelDir(cfg, model, dtype, max_tokens + 1, max_queries)) { fprintf(stderr, "LoadConfig: %s\n", EngineLastError()); return 1; }
    cfg.return_output_tensors_f32 = true;
    cfg.debug.enable_perf_stat = false;
    InferenceEngine engine;
    if (!engine.Init(cfg)) { fprintf(stderr, "Init: %s\n", EngineLastError()); return 1; }
    const int V = engine.VocabSize();
    std::map<std::string, int> ids;            // trace id -> query id
    std::string line;
    while (std::getline(std::cin, line)) {
        if (line.find_first_not_of(" \t\r\n") == std::string::npos) continue;
        JsonValue st; JsonParser jp; std::string err;
        if (!jp.Parse(line, st, &err) || st.type != JsonValue::Object) { fprintf(stderr, "bad step: %s\n", err.c_str()); return 1; }
        long long step = 0;
        st.GetNumber("step", step);
        const JsonValue *entries = st.Get("entries");
        struct Want { int qid; std::vector<int> places; };
        std::vector<Want> wants;
        for (size_t e = 0; entries && e < entries->arr.size(); e++) {
            const JsonValue &en = entries->arr[e];
            std::string id;
            const JsonValue *toks = en.Get("tokens"), *want = en.Get("want");
            if (!en.GetString("id", id) || !toks || toks->arr.empty()) { fprintf(stderr, "step %lld: an entry without id / tokens\n", step); return 1; }
            std::vector<int> t;
            for (const JsonValue &v : toks->arr) t.push_back((int)v.num);
            auto it = ids.find(id);
            int qid;
            if (it == ids.end()) {
                qid = engine.AddQuery(t, QueryOptions());
                if (qid <= 0) { fprintf(stderr, "step %lld: AddQuery: %d %s\n", step, qid, EngineLastError()); return 1; }
                ids[id] = qid;
            } else {
                qid = it->second;
                for (int tok : t) {
                    std::map<int, QueryNextToken> commit; commit[qid].id = tok;
                    if (!engine.CommitInferenceResult(commit)) { fprintf(stderr, "step %lld: Commit: %s\n", step, EngineLastError()); return 1; }
                }
            }
            Want w; w.qid = qid;
            for (size_t k = 0; want && k < want->arr.size(); k++) w.places.push_back((int)want->arr[k].num);
            wants.push_back(w);
        }
        InferenceResult res;
        if (!wants.empty() && !engine.Infer(res)) { fprintf(stderr, "step %lld: Infer: %s\n", step, EngineLastError()); return 1; }
        size_t n_wanted = 0;
        for (const Want &w : wants) n_wanted += w.places.size();
        if (n_wanted) {
            const std::string path = out + "/" + std::to_string(step) + ".f32";
            FILE *fp = fopen(path.c_str(), "wb");
            if (!fp) { fprintf(stderr, "cannot write %s\n", path.c_str()); return 1; }
            for (const Want &w : wants) {
                const QueryInferenceResult *item = nullptr;
                for (const QueryInferenceResult &it : res.items) if (it.query_id == w.qid) item = &it;
                for (int place : w.places) {
                    if (!item || place < 0 || place >= item->output_rows || item->output_cols != V) { fprintf(stderr, "step %lld: no logits for place %d\n", step, place); fclose(fp); return 1; }
                    fwrite(item->output_tensor_f32.data() + (size_t)place * V, 4, (size_t)V, fp);
                }
            }
            fclose(fp);
        }
        if (const JsonValue *end = st.Get("end"))
            for (const JsonValue &v : end->arr) {
                auto it = ids.find(v.str);
                if (it != ids.end()) { engine.RemoveQuery(it->second); ids.erase(it); }
            }
        printf("done %lld\n", step);
        fflush(stdout);
    }
    return 0;
}
