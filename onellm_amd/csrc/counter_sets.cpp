// The process-wide list of counter-set tables (one per kernel family that keeps arrival counters in static device
// memory, in this library and in libonellm_gemm.so) and the two entry points that act on all of them.
#include <algorithm>
#include "counter_sets.hpp"
#include "onellm_hip.h"

namespace onellm {
namespace {
struct TableList {
    std::mutex mu;
    std::vector<CounterSets*> tables;
};
// never destroyed: tables of other libraries unregister from their own static destructors, in an order the
// loader chooses
TableList& table_list()
{
    static TableList* l = new TableList;
    return *l;
}
}  // namespace

void counter_sets_register(CounterSets* table)
{
    TableList& l = table_list();
    std::lock_guard<std::mutex> lock(l.mu);
    l.tables.push_back(table);
}

void counter_sets_unregister(CounterSets* table)
{
    TableList& l = table_list();
    std::lock_guard<std::mutex> lock(l.mu);
    l.tables.erase(std::remove(l.tables.begin(), l.tables.end(), table), l.tables.end());
}

}  // namespace onellm

extern "C" int onellm_release_workspace(const void* workspace)
{
    using namespace onellm;
    if (!workspace) return 0;
    TableList& l = table_list();
    std::lock_guard<std::mutex> lock(l.mu);
    int n = 0;
    for (CounterSets* t : l.tables) n += t->release(workspace);
    return n;
}

extern "C" long onellm_counter_set_fallbacks(void)
{
    using namespace onellm;
    TableList& l = table_list();
    std::lock_guard<std::mutex> lock(l.mu);
    long n = 0;
    for (CounterSets* t : l.tables) n += t->fallbacks();
    return n;
}
