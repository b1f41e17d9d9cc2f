// nart_promark: command-line runner for an engine file — the counterpart of the reference's tools/promark.cpp
// (same options, same JSON configuration, same output file names), built on the art C API only.
//
//   nart_promark -m engine.bin [-c config.json] [-n run_times] [{-i input.bin}] [-s] [-d] [-b batch] [-r name:d0,d1,..] [-y]
//
//   -c  {"workspaces": {"hip": {}, ...}, "input_workspace": "hip"}   (tools/promark.cpp:136-190); every key of
//       "workspaces" names a module: symbol <name>_module_tp, looked up in the process first and then in
//       libart_module_<name>.so (tools/promark.cpp:123-167).  Without -c: {"workspaces": {"default": {}}, ...}.
//   -b  set the batch axis of every input and re-run shape inference (parade_apply_reshape, promark.cpp:329-338)
//   -r  give one input an explicit shape
//   -n  timed runs after two warm-up runs (default 10)
//   -d  fill the inputs with pseudo-random bytes before every timed run
//   -y  time the host<->device copies of inputs and outputs as well
//   -s  after timing: load the -i files into the inputs (in order), run once, write every output tensor to
//       nart-out-<tensor name with '/' -> '_'>.bin
//   -p  (not in the reference) after the timed runs, load the engine p - 1 more times, every copy into workspaces of its
//       own, and time run_times passes handed to the copies in turn without waiting in between: p batches in flight.
//       A GPU workspace owns a stream, so the copies' kernels overlap; the line printed is the time per batch.
//
// Difference from the reference, on purpose: GPU modules run asynchronously, and the reference's timed region
// (promark.cpp:467-476) only waits for the device when -y makes it read an output.  This runner also looks for an
// optional <name>_workspace_synchronize(workspace_t *) in every module and calls it inside the timed region, so
// the reported time is the time of the work, not of its submission.
#include <dlfcn.h>
#include <time.h>
#include <unistd.h>

#include <algorithm>
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "art/art.h"

namespace {

// ---- the small part of JSON the configuration needs: objects, strings, numbers, literals, arrays ----------------
struct Json {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    std::string str;
    double num = 0;
    bool b = false;
    std::vector<Json> arr;
    std::map<std::string, Json> obj; // ordered by key, like the json11 object the reference iterates
    const Json &operator[](const std::string &k) const
    {
        static const Json none;
        auto it = obj.find(k);
        return it == obj.end() ? none : it->second;
    }
};

struct JsonParser {
    const std::string &s;
    size_t i = 0;
    std::string err;
    explicit JsonParser(const std::string &text) : s(text) {}
    void ws()
    {
        while (i < s.size() && std::isspace((unsigned char)s[i]))
            i++;
    }
    bool fail(const char *what)
    {
        if (err.empty())
            err = std::string(what) + " at offset " + std::to_string(i);
        return false;
    }
    bool string(std::string &out)
    {
        if (s[i] != '"')
            return fail("expected '\"'");
        for (i++; i < s.size() && s[i] != '"'; i++) {
            if (s[i] == '\\' && i + 1 < s.size()) {
                const char c = s[++i];
                out += c == 'n' ? '\n' : c == 't' ? '\t' : c == 'r' ? '\r' : c == 'b' ? '\b' : c == 'f' ? '\f' : c;
            } else {
                out += s[i];
            }
        }
        if (i >= s.size())
            return fail("unterminated string");
        i++;
        return true;
    }
    bool value(Json &v, int depth = 0)
    {
        if (depth > 64)
            return fail("nesting too deep");
        ws();
        if (i >= s.size())
            return fail("unexpected end");
        const char c = s[i];
        if (c == '{') {
            v.kind = Json::Object;
            i++;
            ws();
            if (i < s.size() && s[i] == '}') {
                i++;
                return true;
            }
            for (;;) {
                ws();
                std::string key;
                if (i >= s.size() || !string(key))
                    return fail("expected a key");
                ws();
                if (i >= s.size() || s[i] != ':')
                    return fail("expected ':'");
                i++;
                if (!value(v.obj[key], depth + 1))
                    return false;
                ws();
                if (i < s.size() && s[i] == ',') {
                    i++;
                    continue;
                }
                if (i < s.size() && s[i] == '}') {
                    i++;
                    return true;
                }
                return fail("expected ',' or '}'");
            }
        }
        if (c == '[') {
            v.kind = Json::Array;
            i++;
            ws();
            if (i < s.size() && s[i] == ']') {
                i++;
                return true;
            }
            for (;;) {
                v.arr.emplace_back();
                if (!value(v.arr.back(), depth + 1))
                    return false;
                ws();
                if (i < s.size() && s[i] == ',') {
                    i++;
                    continue;
                }
                if (i < s.size() && s[i] == ']') {
                    i++;
                    return true;
                }
                return fail("expected ',' or ']'");
            }
        }
        if (c == '"') {
            v.kind = Json::String;
            return string(v.str);
        }
        if (s.compare(i, 4, "true") == 0) {
            v.kind = Json::Bool, v.b = true, i += 4;
            return true;
        }
        if (s.compare(i, 5, "false") == 0) {
            v.kind = Json::Bool, i += 5;
            return true;
        }
        if (s.compare(i, 4, "null") == 0) {
            i += 4;
            return true;
        }
        char *end = nullptr;
        v.num = strtod(s.c_str() + i, &end);
        if (end == s.c_str() + i)
            return fail("unexpected character");
        v.kind = Json::Number;
        i = (size_t)(end - s.c_str());
        return true;
    }
    bool parse(Json &v)
    {
        if (!value(v))
            return false;
        ws();
        return i == s.size() || fail("trailing characters");
    }
};

// ---- modules and workspaces -----------------------------------------------------------------------------------------
typedef void (*sync_func_t)(workspace_t *);
struct Context {
    std::vector<workspace_t *> ws; // NULL-terminated for the loader
    std::vector<std::string> names;
    std::vector<sync_func_t> sync;
    const mem_tp *input_mem = nullptr;
};

void *find_sym(const std::string &sym, const std::string &lib, bool quiet)
{
    void *p = dlsym(RTLD_DEFAULT, sym.c_str());
    if (p == nullptr && !lib.empty()) {
        void *h = dlopen(lib.c_str(), RTLD_NOW | RTLD_GLOBAL);
        if (h == nullptr) {
            if (!quiet)
                fprintf(stderr, "%s\n", dlerror());
            return nullptr;
        }
        p = dlsym(h, sym.c_str());
        if (p == nullptr && !quiet)
            fprintf(stderr, "%s\n", dlerror());
    }
    return p;
}

bool init_modules(const std::string &config, Context &ctx)
{
    Json json;
    JsonParser parser(config);
    if (!parser.parse(json) || json.kind != Json::Object) {
        fprintf(stderr, "Parse config error: %s\n", parser.err.empty() ? "the top level must be an object" : parser.err.c_str());
        return false;
    }
    const Json &jws = json["workspaces"];
    if (jws.kind != Json::Object) {
        fprintf(stderr, "Parse config error: [workspaces] required\n");
        return false;
    }
    for (const auto &kv : jws.obj) {
        const std::string &name = kv.first;
        const module_t *mod = static_cast<const module_t *>(find_sym(name + "_module_tp", "libart_module_" + name + ".so", false));
        if (mod == nullptr) {
            fprintf(stderr, "[%s] module not found: libart_module_%s.so must be on the library path\n", name.c_str(), name.c_str());
            return false;
        }
        workspace_t *w = workspace_new(mod, nullptr);
        if (w == nullptr) {
            fprintf(stderr, "[%s] the module could not create a workspace\n", name.c_str());
            return false;
        }
        ctx.ws.push_back(w);
        ctx.names.push_back(name);
        ctx.sync.push_back(reinterpret_cast<sync_func_t>(find_sym(name + "_workspace_synchronize", "", true)));
    }
    const Json &jin = json["input_workspace"];
    if (jin.kind != Json::String) {
        fprintf(stderr, "\"input_workspace\" required.\n");
        return false;
    }
    for (size_t i = 0; i < ctx.names.size(); i++)
        if (ctx.names[i] == jin.str)
            ctx.input_mem = workspace_memtype(ctx.ws[i]);
    if (ctx.input_mem == nullptr) {
        fprintf(stderr, "required input workspace [%s] has not been registered.\n", jin.str.c_str());
        return false;
    }
    ctx.ws.push_back(nullptr);
    return true;
}

size_t read_file_chunk(size_t sz, void *data, void *arg) { return fread(data, 1, sz, static_cast<FILE *>(arg)); }

parade_t *load_model(const char *path, const Context &ctx)
{
    FILE *fp = fopen(path, "rb");
    if (fp == nullptr) {
        fprintf(stderr, "cannot open %s\n", path);
        return nullptr;
    }
    buffer_t *buf = nart_buffer_new(0x8000);
    buffer_set_buffer_read_func(buf, read_file_chunk, fp);
    deserialize_param_t params = {ctx.ws.data(), ctx.input_mem};
    parade_t *model = deserialize_parade(buf, &params);
    nart_buffer_delete(buf);
    fclose(fp);
    if (model != nullptr)
        parade_prepare(model);
    return model;
}

const char *dtype_name(uint32_t tp)
{
    switch (tp) {
    case dtFLOAT32: return "FLOAT32";
    case dtFLOAT16: return "FLOAT16";
    case dtINT32: return "INT32";
    case dtINT16: return "INT16";
    case dtINT8: return "INT8";
    case dtUINT32: return "UINT32";
    case dtUINT16: return "UINT16";
    case dtUINT8: return "UINT8";
    default: return "UNKNOWN";
    }
}

size_t tensor_bytes(const tensor_t *t) { return shape_count(&t->shape) * datatype_sizeof(t->dtype); }

void print_tensors(const char *title, size_t n, tensor_array_t ts)
{
    printf("%s:\n", title);
    for (size_t i = 0; i < n; i++) {
        printf("\t%s:  %s %u", ts[i]->name ? ts[i]->name : "(unnamed)", dtype_name(ts[i]->dtype), ts[i]->shape.dim[0]);
        for (int j = 1; j < ts[i]->shape.dim_size; j++)
            printf(", %u", ts[i]->shape.dim[j]);
        printf("\n");
    }
}

bool load_input(const char *path, tensor_t *t)
{
    void *data = mem_cpu_data(t->mem);
    const size_t size = tensor_bytes(t);
    FILE *fp = fopen(path, "rb");
    if (fp == nullptr) {
        fprintf(stderr, "cannot open %s\n", path);
        return false;
    }
    const size_t got = fread(data, 1, size, fp);
    fclose(fp);
    if (got != size)
        fprintf(stderr, "%s holds %zu bytes, tensor %s needs %zu\n", path, got, t->name ? t->name : "?", size);
    return got == size;
}

bool save_output(const char *path, tensor_t *t)
{
    const void *data = mem_cpu_data(t->mem); // downloads what the device holds
    const size_t size = tensor_bytes(t);
    FILE *fp = fopen(path, "wb");
    if (fp == nullptr)
        return false;
    const size_t put = fwrite(data, 1, size, fp);
    fclose(fp);
    return put == size;
}

double now_ms()
{
    timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return ts.tv_sec * 1e3 + ts.tv_nsec * 1e-6;
}

int usage(const char *argv0)
{
    fprintf(stderr, "Usage: \n%s -m model [-c config] [-n run_times] [{-i blob.bin}] [-s] [-d] [-b batch_size] [-r name:d0,d1,...] [-y] [-p parades_in_flight]\n",
            argv0);
    return 1;
}

} // namespace

int main(int argc, char *argv[])
{
    if (argc == 1)
        return usage(argv[0]);
    std::string model_file, config_file;
    int run_times = 10, batch_size = -1, in_flight = 1;
    std::vector<std::string> inputs;
    bool save_flag = false, randomized = false, with_copies = false;
    std::map<std::string, std::vector<int>> shape_by_name;
    int ch;
    while ((ch = getopt(argc, argv, "i:sm:c:n:b:r:dyp:")) != -1) {
        switch (ch) {
        case 'm': model_file = optarg; break;
        case 'c': config_file = optarg; break;
        case 'n': run_times = atoi(optarg); break;
        case 'i': inputs.push_back(optarg); break;
        case 'b': batch_size = atoi(optarg); break;
        case 's': save_flag = true; break;
        case 'd': randomized = true; break;
        case 'y': with_copies = true; break;
        case 'p': in_flight = atoi(optarg); break;
        case 'r': {
            const std::string arg(optarg);
            const size_t pos = arg.find(':');
            if (pos == std::string::npos)
                break;
            std::vector<int> shape;
            size_t p = pos + 1;
            while (p < arg.size()) {
                size_t q = arg.find(',', p);
                if (q == std::string::npos)
                    q = arg.size();
                if (q > p)
                    shape.push_back(atoi(arg.substr(p, q - p).c_str()));
                p = q + 1;
            }
            shape_by_name[arg.substr(0, pos)] = shape;
            break;
        }
        default: return usage(argv[0]);
        }
    }
    if (model_file.empty() || run_times < 0 || in_flight < 1 || in_flight > 8)
        return usage(argv[0]);
    printf("parse args ...\n  modelfile  : %s\n  config_file: %s\n  run_time   : %d\n\n", model_file.c_str(), config_file.c_str(),
           run_times);

    std::string config = "{\"workspaces\": {\"default\": {}}, \"input_workspace\": \"default\"}";
    if (!config_file.empty()) {
        FILE *fp = fopen(config_file.c_str(), "rb");
        if (fp != nullptr) {
            config.clear();
            char chunk[4096];
            size_t n;
            while ((n = fread(chunk, 1, sizeof chunk, fp)) > 0)
                config.append(chunk, n);
            fclose(fp);
        }
    }
    Context ctx;
    if (!init_modules(config, ctx)) {
        fprintf(stderr, "init module failed!\n");
        return 1;
    }
    parade_t *parade = load_model(model_file.c_str(), ctx);
    if (parade == nullptr) {
        fprintf(stderr, "loading %s failed\n", model_file.c_str());
        return 1;
    }
    size_t input_cnt = 0, output_cnt = 0;
    tensor_array_t in_t = nullptr, out_t = nullptr;
    if (!parade_get_input_tensors(parade, &input_cnt, &in_t) || !parade_get_output_tensors(parade, &output_cnt, &out_t)) {
        fprintf(stderr, "the engine has no input / output table\n");
        return 1;
    }

    auto reshape = [&](parade_t *pa, size_t n_in, tensor_array_t tin) {
        if (batch_size > 0) {
            for (size_t i = 0; i < n_in; i++)
                tin[i]->shape.dim[tin[i]->shape.batch_axis] = (uint32_t)batch_size;
            if (!parade_apply_reshape(pa))
                return false;
        }
        if (!shape_by_name.empty()) {
            for (size_t i = 0; i < n_in; i++) {
                auto it = tin[i]->name ? shape_by_name.find(tin[i]->name) : shape_by_name.end();
                if (it == shape_by_name.end())
                    continue;
                tin[i]->shape.dim_size = (int32_t)it->second.size();
                for (size_t d = 0; d < it->second.size() && d < 8; d++)
                    tin[i]->shape.dim[d] = (uint32_t)it->second[d];
            }
            if (!parade_apply_reshape(pa))
                return false;
        }
        return true;
    };
    if (!reshape(parade, input_cnt, in_t)) {
        fprintf(stderr, "Reshape parade failed\n");
        return 1;
    }
    print_tensors("input tensors", input_cnt, in_t);
    print_tensors("output tensors", output_cnt, out_t);

    auto sync_all = [&]() {
        for (size_t i = 0; i + 1 < ctx.ws.size(); i++)
            if (ctx.sync[i])
                ctx.sync[i](ctx.ws[i]);
    };
    for (size_t i = 0; i < input_cnt; i++)
        memset(mem_cpu_data(in_t[i]->mem), 0, tensor_bytes(in_t[i]));
    printf("\nWarming up ...\n");
    parade_run(parade);
    parade_run(parade);
    sync_all();
    printf("\nFinish warm up\n");

    double total = 0;
    unsigned rng = 12345u;
    for (int it = 0; it < run_times; it++) {
        if (randomized) {
            printf("use randomized data.\n");
            for (size_t j = 0; j < input_cnt; j++) {
                unsigned char *p = static_cast<unsigned char *>(mem_cpu_data(in_t[j]->mem));
                const size_t n = tensor_bytes(in_t[j]);
                for (size_t k = 0; k < n; k++) {
                    rng = rng * 1664525u + 1013904223u;
                    p[k] = (unsigned char)(rng >> 24);
                }
            }
        }
        if (with_copies) { // leave the inputs dirty on the host side so that the run uploads them
            for (size_t j = 0; j < input_cnt; j++)
                (void)mem_cpu_data(in_t[j]->mem);
        } else { // upload now, outside the timed region
            for (size_t j = 0; j < input_cnt; j++)
                (void)mem_data(in_t[j]->mem);
            sync_all();
        }
        const double t0 = now_ms();
        parade_run(parade);
        if (with_copies)
            for (size_t j = 0; j < output_cnt; j++)
                (void)mem_cpu_data(out_t[j]->mem);
        sync_all();
        const double dt = now_ms() - t0;
        total += dt;
        printf("Process %d : cost %gms\n", it, dt);
    }
    if (run_times > 0)
        printf("\nTest finised, average cost: %gms\n\n", total / run_times);

    // ---- -p: several parades in flight -----------------------------------------------------------------------
    std::vector<Context> more_ctx((size_t)in_flight - 1);
    std::vector<parade_t *> parades(1, parade);
    for (int k = 1; k < in_flight; k++) {
        Context &c = more_ctx[(size_t)k - 1];
        parade_t *pa = init_modules(config, c) ? load_model(model_file.c_str(), c) : nullptr;
        size_t n_in = 0;
        tensor_array_t tin = nullptr;
        if (pa == nullptr || !parade_get_input_tensors(pa, &n_in, &tin) || !reshape(pa, n_in, tin)) {
            fprintf(stderr, "loading copy %d of the engine failed\n", k);
            return 1;
        }
        for (size_t i = 0; i < n_in; i++) {
            memset(mem_cpu_data(tin[i]->mem), 0, tensor_bytes(tin[i]));
            (void)mem_data(tin[i]->mem); // upload outside the timed region
        }
        parade_run(pa);
        parades.push_back(pa);
    }
    if (in_flight > 1 && run_times > 0) {
        auto sync_every = [&]() {
            sync_all();
            for (Context &c : more_ctx)
                for (size_t i = 0; i + 1 < c.ws.size(); i++)
                    if (c.sync[i])
                        c.sync[i](c.ws[i]);
        };
        for (size_t j = 0; j < input_cnt; j++)
            (void)mem_data(in_t[j]->mem);
        for (int it = 0; it < 2 * in_flight; it++)
            parade_run(parades[(size_t)(it % in_flight)]);
        sync_every();
        const double t0 = now_ms();
        for (int it = 0; it < run_times; it++)
            parade_run(parades[(size_t)(it % in_flight)]);
        sync_every();
        printf("%d parades in flight, %d passes: average cost per batch: %gms\n\n", in_flight, run_times,
               (now_ms() - t0) / run_times);
    }

    int rc = 0;
    if (save_flag) {
        if (inputs.size() != input_cnt) {
            fprintf(stderr, "Warning: Inputs file mismatch with model's inputs, which requires %zu, but given %zu\n", input_cnt,
                    inputs.size());
        } else {
            for (size_t i = 0; i < input_cnt; i++)
                if (!load_input(inputs[i].c_str(), in_t[i]))
                    rc = 1;
        }
        parade_run(parade);
        fprintf(stderr, "Info: Saving output tensors ...\n");
        for (size_t i = 0; i < output_cnt; i++) {
            std::string name = out_t[i]->name ? out_t[i]->name : "output" + std::to_string(i);
            std::replace(name.begin(), name.end(), '/', '_');
            if (!save_output(("nart-out-" + name + ".bin").c_str(), out_t[i]))
                rc = 1;
        }
    }
    for (parade_t *pa : parades)
        parade_delete(pa);
    for (size_t i = 0; i + 1 < ctx.ws.size(); i++)
        workspace_delete(ctx.ws[i]);
    for (Context &c : more_ctx)
        for (size_t i = 0; i + 1 < c.ws.size(); i++)
            workspace_delete(c.ws[i]);
    return rc;
}
