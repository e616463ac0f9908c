// Command-line generator with the reference's five positional arguments
// (cogent/tc_code_generator.py:13-25, as invoked by cogent/tccg.sh:43):
//
//   cogent_gen <number> <input.in> <config# or -1> <pre_computed: -1 or 1> <DOUBLE or FLOAT>
//
// and writes temp__<number>.hip into the working directory, where the reference
// writes temp__<number>.cu (cogent/src/codes/tc_gen_code.py:27-30).  The
// pre-computed-array switch is accepted and ignored: addresses are always
// computed inside the kernel.  Extra options: -o <path>, --name <unique>,
// --map <spec>, --json (print the plan), --list <k> (print the k cheapest mappings).
#include "../../include/cogent_mi355.h"
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

int main(int argc, char** argv)
{
    std::vector<std::string> pos;
    std::string out_path, name, spec;
    bool want_json = false;
    int list_k = 0;
    for (int i = 1; i < argc; i++) {
        std::string a = argv[i];
        if (a == "-o" && i + 1 < argc) out_path = argv[++i];
        else if (a == "--name" && i + 1 < argc) name = argv[++i];
        else if (a == "--map" && i + 1 < argc) spec = argv[++i];
        else if (a == "--json") want_json = true;
        else if (a == "--list" && i + 1 < argc) list_k = atoi(argv[++i]);
        else pos.push_back(a);
    }
    if (pos.size() != 5) {
        fprintf(stderr, "[Code Generator] Please check arguments...\n"
                        "usage: cogent_gen <number> <input.in> <config# or -1> <pre_computed: -1 or 1> <DOUBLE or FLOAT> [-o out.hip] [--name id] [--map spec] [--json] [--list k]\n");
        return 2;
    }
    std::ifstream f(pos[1]);
    if (!f) { fprintf(stderr, "cannot open %s\n", pos[1].c_str()); return 1; }
    std::stringstream ss;
    ss << f.rdbuf();
    if (name.empty()) name = "tc_" + pos[0];
    if (out_path.empty()) out_path = "temp__" + pos[0] + ".hip";
    // several expressions in one file: a fused group (they must share the output), one kernel for all
    {
        int n_expr = 0;
        std::istringstream lines(ss.str());
        std::string line;
        while (std::getline(lines, line)) {
            size_t p = line.find_first_not_of(" \t\r");
            if (p != std::string::npos && line[p] != '#') n_expr++;
        }
        if (n_expr > 1) {
            int rc = cogent_group_emit(ss.str().c_str(), pos[4].c_str(), spec.empty() ? nullptr : spec.c_str(), name.c_str(), out_path.c_str());
            if (rc) { fprintf(stderr, "cogent_gen: %s\n", cogent_host_last_error()); return rc; }
            if (want_json) printf("%s\n", cogent_group_last_json());
            return 0;
        }
    }
    cogent_plan* plan = nullptr;
    int rc = cogent_plan_create(ss.str().c_str(), pos[4].c_str(), atoi(pos[2].c_str()), spec.empty() ? nullptr : spec.c_str(), &plan);
    if (rc) { fprintf(stderr, "cogent_gen: %s\n", cogent_host_last_error()); return rc; }
    if (want_json) printf("%s\n", cogent_plan_json(plan));
    if (list_k > 0) printf("%s\n", cogent_plan_candidates_json(plan, list_k));
    rc = cogent_plan_emit(plan, name.c_str(), out_path.c_str());
    if (rc) fprintf(stderr, "cogent_gen: %s\n", cogent_host_last_error());
    cogent_plan_destroy(plan);
    return rc;
}
