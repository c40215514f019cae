// Drives every xft::Model::set_input overload of include/models.h (the reference's include/models.h:40-73)
// and Model::forward through the C++ API, the way a program written against the reference's header would:
//     set_input_driver <model directory> <dtype> <vocab>
// Every sequence, whichever overload made it, must continue greedily as it does alone through
// input() / config() / generate().  Prints one line per check and the lockstep ids (for the caller to compare
// with another binding); exit status 0 only if every check passed.  Built by xfastertransformer_amd/build.py.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "models.h"

static int failures = 0;

static void check(bool ok, const char *what) {
    printf("%s %s\n", ok ? "OK  " : "FAIL", what);
    if (!ok) ++failures;
}

static std::vector<int32_t> prompt_of(int n, int salt, int vocab) {
    std::vector<int32_t> p(n);
    unsigned long long s = 88172645463325252ull + (unsigned)salt * 7919u;
    for (int i = 0; i < n; ++i) {
        s ^= s << 13, s ^= s >> 7, s ^= s << 17;
        p[i] = (int32_t)(s % (unsigned)vocab);
    }
    return p;
}

static int argmax_row(const float *row, int vocab) {
    int best = 0;
    for (int j = 1; j < vocab; ++j)
        if (row[j] > row[best]) best = j;
    return best;
}

int main(int argc, char **argv) {
    if (argc < 4) {
        fprintf(stderr, "usage: %s <model dir> <dtype> <vocab>\n", argv[0]);
        return 2;
    }
    const std::string path = argv[1], dtype = argv[2];
    const int vocab = atoi(argv[3]);
    const xft::DataType dt = dtype == "int8" ? xft::DataType::int8 : dtype == "int4" ? xft::DataType::int4 : xft::DataType::bf16;
    xft::AutoModel model(path, dt);
    check(model.getVocabSize() == vocab, "vocabulary size");
    const int never = vocab + 5, gen = 6;
    const std::vector<std::vector<int32_t>> prompts = {prompt_of(7, 1, vocab), prompt_of(7, 2, vocab), prompt_of(12, 3, vocab)};

    // what every sequence generates alone (lockstep API)
    std::vector<std::vector<int32_t>> alone;
    for (const auto &p : prompts) {
        std::vector<int32_t> ids = p;
        model.config((int)p.size() + gen, 1, 1, 1.0f, false, never);
        model.input(ids, 1);
        while (!model.isDone()) model.generate();
        std::vector<int32_t> out = model.finalize();
        alone.emplace_back(out.begin() + p.size(), out.end());
        printf("ALONE");
        for (int t : alone.back()) printf(" %d", t);
        printf("\n");
    }
    auto continues = [&](int k, const std::vector<int32_t> &got) {
        if (got.size() > alone[k].size()) return false;
        for (size_t i = 0; i < got.size(); ++i)
            if (got[i] != alone[k][i]) return false;
        return !got.empty();
    };
    // runs the working sequences through generate() until done, returns prompt + generated back to back
    auto run_generate = [&]() {
        while (!model.isDone()) model.generate();
        return model.finalize();
    };
    auto split_two = [&](const std::vector<int32_t> &flat, size_t len0) {
        return std::make_pair(std::vector<int32_t>(flat.begin() + 7, flat.begin() + len0), std::vector<int32_t>(flat.begin() + len0 + 7, flat.end()));
    };
    std::vector<int32_t> flat01 = prompts[0];
    flat01.insert(flat01.end(), prompts[1].begin(), prompts[1].end());

    {   // (ids, batch, maxLen, ...): flat arguments
        std::vector<int> ids = model.set_input(flat01, 2, 7 + gen, 1, 1, 1.0f, false, never);
        check(ids.size() == 2 && ids[0] != ids[1], "set_input(ids, batch, maxLen, ...) returns two ids");
        auto out = run_generate();
        auto parts = split_two(out, out.size() / 2);
        check(out.size() == 2 * (7 + gen) && continues(0, parts.first) && continues(1, parts.second), "  ... generates what each prompt does alone");
    }
    {   // (ids, batch, SearcherConfig)
        SearcherConfig cfg(7 + gen);
        cfg.eosTokenId = never;
        std::vector<int> ids = model.set_input(flat01, 2, cfg);
        auto out = run_generate();
        auto parts = split_two(out, out.size() / 2);
        check(ids.size() == 2 && continues(0, parts.first) && continues(1, parts.second), "set_input(ids, batch, config)");
    }
    {   // (prompts, SearcherConfig) with ragged prompts, then (prompts, seqIDs, SearcherConfig) selecting one of them
        SearcherConfig cfg(12 + gen);
        cfg.eosTokenId = never;
        std::vector<std::vector<int32_t>> two = {prompts[0], prompts[2]};
        std::vector<int> ids = model.set_input(two, cfg);
        std::vector<int32_t> first = model.generate(); // the prompts
        std::vector<std::vector<int32_t>> got = {{first[0]}, {first[1]}};
        std::vector<std::vector<int32_t>> none = {{0}};
        for (int step = 0; step < 2; ++step) { // only the second sequence steps
            std::vector<int> sel = {ids[1]};
            model.set_input(none, sel, cfg);
            got[1].push_back(model.generate()[0]);
        }
        std::vector<std::vector<int32_t>> none2 = {{0}, {0}};
        model.set_input(none2, ids, cfg);
        std::vector<int32_t> both = model.generate();
        got[0].push_back(both[0]), got[1].push_back(both[1]);
        check(ids.size() == 2 && continues(0, got[0]) && continues(2, got[1]) && got[1].size() == 4, "set_input(prompts, config) + set_input(prompts, seqIDs, config)");
        check(model.freeSeqs(ids) && !model.freeSeqs(ids), "freeSeqs");
    }
    {   // (prompts, maxLen, ...): flat arguments, ragged prompts
        std::vector<std::vector<int32_t>> two = {prompts[2], prompts[1]};
        std::vector<int> ids = model.set_input(two, 12 + gen, 1, 1, 1.0f, false, never);
        std::vector<int32_t> t0 = model.generate();
        std::vector<std::vector<int32_t>> none = {{0}, {0}};
        SearcherConfig cfg = model.getConfig();
        model.set_input(none, ids, cfg);
        std::vector<int32_t> t1 = model.generate();
        check(continues(2, {t0[0], t1[0]}) && continues(1, {t0[1], t1[1]}), "set_input(prompts, maxLen, ...)");
        model.freeSeqs(ids);
    }
    // ---- the forms that go with forward(): the caller picks the tokens ----
    auto drive_forward = [&](std::vector<int> ids, const std::vector<int> &which, std::vector<std::vector<int32_t>> &got, int form) {
        // one decode step of sequences `ids` (tokens: the last of got[]), through set_input form 0..3
        std::vector<int32_t> toks;
        for (size_t i = 0; i < ids.size(); ++i) toks.push_back(got[which[i]].back());
        if (form == 0) {
            std::vector<std::vector<int32_t>> in;
            for (int t : toks) in.push_back({t});
            model.set_input(in, ids, -1);
        } else if (form == 1) {
            model.set_input(toks, (int)toks.size(), ids, -1);
        } else if (form == 2) {
            const std::vector<int> maxLen;
            model.set_input(toks, (int)toks.size(), ids, maxLen);
        } else {
            std::vector<int32_t> lens;
            std::vector<int> maxLen;
            model.set_input(toks, lens, ids, maxLen);
        }
        auto r = model.forward(false);
        if (std::get<1>(r) != (int)ids.size() || std::get<2>(r) != vocab) return false;
        for (size_t i = 0; i < ids.size(); ++i) got[which[i]].push_back(argmax_row(std::get<0>(r) + i * (size_t)vocab, vocab));
        return true;
    };
    for (int form = 0; form < 4; ++form) {
        std::vector<int> ids;
        std::vector<std::vector<int32_t>> got(3);
        bool ok = true;
        std::tuple<float *, int, int> r;
        if (form == 0) { // (prompts, seqIDs = {}, maxLen): ragged
            std::vector<std::vector<int32_t>> in = {prompts[0], prompts[2]};
            ids = model.set_input(in, std::vector<int> {}, 12 + gen + 2); // (a bare {} would pick the flat-argument form)
            r = model.forward(false);
            ok = std::get<1>(r) == 2;
            got[0].push_back(argmax_row(std::get<0>(r), vocab)), got[2].push_back(argmax_row(std::get<0>(r) + vocab, vocab));
        } else if (form == 1 || form == 2) { // (ids, batch, seqIDs = {}, maxLen) / (..., vector maxLen): equal lengths
            std::vector<int32_t> in = flat01;
            if (form == 1) ids = model.set_input(in, 2, std::vector<int> {}, 7 + gen + 2);
            else ids = model.set_input(in, 2, std::vector<int> {}, std::vector<int> {7 + gen + 2, 7 + gen + 3});
            r = model.forward(false);
            ok = std::get<1>(r) == 2;
            got[0].push_back(argmax_row(std::get<0>(r), vocab)), got[1].push_back(argmax_row(std::get<0>(r) + vocab, vocab));
        } else { // (ids, seqLens, seqIDs, maxLen): ragged, back to back; logits of every position
            std::vector<int32_t> in = prompts[2];
            in.insert(in.end(), prompts[0].begin(), prompts[0].end());
            std::vector<int32_t> lens = {12, 7};
            std::vector<int> maxLen = {30};
            ids = model.set_input(in, lens, std::vector<int> {}, maxLen);
            r = model.forward(true);
            ok = std::get<1>(r) == 19 && std::get<2>(r) == vocab;
            got[2].push_back(argmax_row(std::get<0>(r) + (size_t)11 * vocab, vocab));
            got[0].push_back(argmax_row(std::get<0>(r) + (size_t)18 * vocab, vocab));
        }
        const std::vector<int> which = form == 0 ? std::vector<int> {0, 2} : form == 3 ? std::vector<int> {2, 0} : std::vector<int> {0, 1};
        for (int step = 0; step < 3 && ok; ++step) ok = drive_forward(ids, which, got, form);
        // one sequence alone for a step, then both again
        if (ok) ok = drive_forward({ids[1]}, {which[1]}, got, form) && drive_forward(ids, which, got, form);
        for (int k : which) ok = ok && continues(k, got[k]);
        ok = ok && got[which[1]].size() == 6 && got[which[0]].size() == 5;
        char name[96];
        snprintf(name, sizeof(name), "forward-only set_input form %d + forward()", form);
        check(ok, name);
        check(model.freeSeqs(ids), "  freeSeqs of its sequences");
    }
    // the lockstep API still works after the sequence-id interface
    {
        std::vector<int32_t> ids = prompts[1];
        model.config(7 + gen, 1, 1, 1.0f, false, never);
        model.input(ids, 1);
        auto r = model.forward(false);
        check(std::get<1>(r) == 0 && argmax_row(std::get<0>(r), vocab) == alone[1][0], "input() + forward(false)");
        auto all = model.forward(true);
        check(argmax_row(std::get<0>(all) + (size_t)6 * vocab, vocab) == alone[1][0], "input() + forward(true): last row");
    }
    printf("%s\n", failures ? "FAILED" : "PASSED");
    return failures ? 1 : 0;
}
