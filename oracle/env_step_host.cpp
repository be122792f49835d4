/*
 * Host build of the library's env step.  TEST INFRASTRUCTURE ONLY.
 *
 * craftax.cu_amd/csrc/env_logic.h is the text the gfx950 kernel compiles; here the same
 * text is compiled for the host over a plain cfp_env_state (HostStore of env_host.h), so
 * that the game logic can be held to the compiled reference (oracle/_ref) field by field
 * without a GPU, and so that a difference on the GPU can be told apart from one in the
 * logic.  Nothing in the product library links or loads this file.
 * Output: oracle/libcfenvhost.so.  Strict fp32: built with -ffp-contract=off.
 */
#include "../craftax.cu_amd/csrc/env_host.h"

extern "C" {

size_t cfhost_state_bytes(void) { return sizeof(cfp_env_state); }

void cfhost_light_table(float* out, int count) {
    for (int t = 0; t < count; t++) out[t] = cfenv::light_level(t);
}

/* One step of each of `count` states with the given actions. */
void cfhost_step(cfp_env_state* states, int count, const float* actions, const float* light,
                 float* rewards, float* terminals, uint32_t* reset_keys /* [count][2] */) {
    for (int i = 0; i < count; i++)
        cfenv::host_step(states[i], actions[i], light, &rewards[i], &terminals[i], &reset_keys[2 * i]);
}

/* States of envs created with seeds seed0, seed0 + 1, ... (c_init), generated on the host. */
void cfhost_generate(uint32_t seed0, int count, cfp_env_state* states) {
    static cfenv::FloorScratch sc;
    for (int i = 0; i < count; i++) cfenv::generate_env_host(seed0 + (uint32_t)i, states[i], sc);
}
/* The state a finished env is reset to from its reset key. */
void cfhost_reset(cfp_env_state* state, const uint32_t reset_key[2]) {
    static cfenv::FloorScratch sc;
    cfenv::generate_world_host(cfenv::world_key_of_reset((uint64_t)reset_key[1] << 32 | reset_key[0]), *state, sc);
}

void cfhost_derive_spawn_planes(cfp_env_state* states, int count) {
    for (int i = 0; i < count; i++) cfenv::derive_spawn_planes(states[i]);
}

}  /* extern "C" */
