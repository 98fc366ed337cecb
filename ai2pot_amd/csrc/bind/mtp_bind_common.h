// Shared by libmtpr_bind.so and libnnmtp_bind.so (each gets its own copy of the state): the
// template-file parser behind mtpParamOp (source/descriptor/mtpr/src/mtpParam.cc:32-43, 65-214,
// 435-469; the nnmtp copy of that file is identical) and the cache of contraction plans.
#pragma once
#include "bind_common.h"

#include <cstdlib>
#include <fstream>
#include <map>
#include <mutex>
#include <regex>
#include <set>
#include <sstream>
#include <tuple>

using namespace a2p_bind;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

namespace {

std::string g_ai2pot_path;

// ---- template files (source/descriptor/mtpr/src/mtpParam.cc:32-43, 65-214) ---------------------
std::string template_dir()
{
    const char* env = std::getenv("AI2POT_PATH");
    if (env) return std::string(env) + "/source/descriptor/mtpr/MTP_templates/";
    return g_ai2pot_path + "/_data/MTP_templates/";
}

struct Tables {
    int n_moms = 0;
    std::vector<int> basic, times, mapping;     // flattened [n,4], [n,4], [n]
};

std::vector<int> ints_after(const std::string& body, const std::string& key)
{
    std::regex re("(^|\\n)\\s*" + key + "\\s*=\\s*([^\\n]*)");
    std::smatch m;
    TORCH_CHECK(std::regex_search(body, m, re), "Cannot read ", key, ".");
    std::vector<int> out;
    const std::string line = m[2];
    std::regex num("-?\\d+");
    for (auto it = std::sregex_iterator(line.begin(), line.end(), num); it != std::sregex_iterator(); ++it)
        out.push_back(std::stoi(it->str()));
    return out;
}

Tables load_tables(int level)
{
    TORCH_CHECK(level >= 2 && level <= 28 && level % 2 == 0, "mtp level must be an even number in 2..28");
    std::string name = level <= 4 ? "depreciated-0" + std::to_string(level) + ".almtp"
                                  : (level < 10 ? "0" : "") + std::to_string(level) + ".almtp";
    const std::string path = template_dir() + name;
    std::ifstream ifs(path);
    TORCH_CHECK(ifs.is_open(), "Cannot open file ", path);
    std::string line, body;
    for (int i = 0; i < 10; i++) std::getline(ifs, line);        // header is ignored, mtpParam.cc:92-93
    std::stringstream ss;
    ss << ifs.rdbuf();
    body = ss.str();
    Tables t;
    auto one = [&](const char* key) {
        auto v = ints_after(body, key);
        TORCH_CHECK(v.size() == 1, "Cannot read ", key, ".");
        return v[0];
    };
    t.n_moms = one("alpha_moments_count");
    const int nb = one("alpha_index_basic_count"), nt = one("alpha_index_times_count"),
              ns = one("alpha_scalar_moments");
    t.basic = ints_after(body, "alpha_index_basic");
    t.times = nt ? ints_after(body, "alpha_index_times") : std::vector<int>();
    t.mapping = ints_after(body, "alpha_moment_mapping");
    TORCH_CHECK((int)t.basic.size() == 4 * nb, "Cannot read alpha_index_basic.");
    TORCH_CHECK((int)t.times.size() == 4 * nt, "Cannot read alpha_index_times.");
    TORCH_CHECK((int)t.mapping.size() == ns, "Cannot read alpha_moment_mapping.");
    return t;
}

variable_list mtp_param_op(int64_t level)
{
    Tables t = load_tables((int)level);
    const int nb = (int)t.basic.size() / 4, nt = (int)t.times.size() / 4;
    // radial-function indices each moment depends on (mtpParam.cc:435-469)
    std::vector<std::set<int>> mus(t.n_moms);
    for (int i = 0; i < nb && i < t.n_moms; i++) mus[i].insert(t.basic[i * 4]);
    for (int i = nb; i < t.n_moms; i++)
        for (int e = 0; e < nt; e++)
            if (t.times[e * 4 + 3] == i) {
                const auto &a = mus[t.times[e * 4]], &b = mus[t.times[e * 4 + 1]];
                mus[i].insert(a.begin(), a.end());
                mus[i].insert(b.begin(), b.end());
            }
    size_t width = 0;
    int nmus = 1;
    for (auto& s : mus) width = std::max(width, s.size());
    for (int i = 0; i < nb; i++) nmus = std::max(nmus, t.basic[i * 4] + 1);
    auto iopt = at::TensorOptions().dtype(at::kInt);
    at::Tensor basic = at::from_blob(t.basic.data(), {nb, 4}, iopt).clone();
    at::Tensor times = nt ? at::from_blob(t.times.data(), {nt, 4}, iopt).clone() : at::zeros({0, 4}, iopt);
    at::Tensor mapping = at::from_blob(t.mapping.data(), {(int64_t)t.mapping.size()}, iopt).clone();
    at::Tensor num = at::zeros({t.n_moms}, iopt);
    at::Tensor m4m = at::zeros({t.n_moms, (int64_t)width}, iopt) - 1;
    for (int i = 0; i < t.n_moms; i++) {
        num.data_ptr<int>()[i] = (int)mus[i].size();
        int c = 0;
        for (int v : mus[i]) m4m.data_ptr<int>()[i * width + (c++)] = v;
    }
    return {torch::tensor(t.n_moms, iopt), basic, times, mapping, num, m4m, torch::tensor(nmus, iopt)};
}

// ---- plan cache ---------------------------------------------------------------------------------
struct PlanEntry {
    void* handle;
    int n_scalar;
};
std::mutex g_plan_mutex;
std::map<std::tuple<int, int64_t, const void*, int64_t, uint32_t, const void*, int64_t, uint32_t, const void*,
                    int64_t, uint32_t>, PlanEntry> g_plans;

PlanEntry get_plan(int device, int64_t n_moms, const at::Tensor& basic, const at::Tensor& times,
                   const at::Tensor& mapping)
{
    // the tables are model constants (registered buffers, ai2pot/models/mtp/linear_mtp.py:63-69):
    // read back once, cached by storage address, size and version
    auto key = std::make_tuple(device, n_moms, basic.data_ptr(), basic.numel(), basic._version(),
                               times.data_ptr(), times.numel(), times._version(), mapping.data_ptr(),
                               mapping.numel(), mapping._version());
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    auto it = g_plans.find(key);
    if (it != g_plans.end()) return it->second;
    for (auto* t : {&basic, &times, &mapping})
        TORCH_CHECK(t->scalar_type() == at::kInt, "the MTP index tensors must be int32");
    TORCH_CHECK(basic.dim() == 2 && basic.size(1) == 4, "alpha_index_basic must have shape [n, 4]");
    TORCH_CHECK(times.numel() == 0 || (times.dim() == 2 && times.size(1) == 4),
                "alpha_index_times must have shape [n, 4]");
    at::Tensor hb = basic.cpu().contiguous(), ht = times.cpu().contiguous(), hm = mapping.cpu().contiguous();
    PlanEntry e;
    e.n_scalar = (int)hm.numel();
    check_rc(a2p_mtp_plan_create((int)n_moms, (int)hb.size(0), hb.data_ptr<int>(), (int)(ht.numel() / 4),
                                 ht.numel() ? ht.data_ptr<int>() : nullptr, e.n_scalar, hm.data_ptr<int>(),
                                 &e.handle));
    g_plans[key] = e;
    return e;
}

}  // namespace
