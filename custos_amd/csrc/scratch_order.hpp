// Who has to wait for whom on a GPU's shared operand table (custos_hip_apply_fn_many_noalloc).
//
// All handles on a GPU share that GPU's table, each launching on a stream of its own.  A call
// rewrites the table and then launches a grid that reads it, so it must not start before the last
// grid that read the table has finished.  Calls through one handle are ordered by its stream; for
// calls through different handles there is one event per GPU, recorded behind a launch and waited
// for by the next caller's stream.  While a GPU has a single handle nothing needs recording; when
// a second handle appears the event is recorded once behind whatever the table's last user has
// launched so far, and from then on behind every launch.
//
// This class only decides; the caller issues the event calls under the mutex that guards it.  No
// HIP types: the decisions are tested on the host against a model of streams and events.
#pragma once

namespace custos_hip {

struct ScratchOrder {
    const void* last_user = nullptr;  // the handle whose launch read the table last (null: nobody, or it has finished)
    int handles = 0;                  // handles alive on this GPU

    // A handle appears.  True: record the event now on `last_user`'s stream.
    bool handle_created() { return ++handles == 2 && last_user != nullptr; }
    // (when that recording fails the handle does not take part)
    void handle_not_created() { --handles; }
    // A handle goes away, after its stream has drained.
    void handle_destroyed(const void* handle) {
        if (last_user == handle) last_user = nullptr;
        --handles;
    }
    // Before `handle` rewrites the table.  True: its stream first waits for the event.
    bool must_wait(const void* handle) const { return last_user != nullptr && last_user != handle; }
    // Whether nobody but `handle` has used the table since `handle` used it last (what it sent is still there).
    bool still_holds_rows_of(const void* handle) const { return last_user == handle; }
    // After `handle` launched the grid that reads the table.  True: record the event behind it.
    bool launched(const void* handle) {
        last_user = handle;
        return handles > 1;
    }
};

}  // namespace custos_hip
