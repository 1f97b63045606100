// Random numbers of devices::ROCM (the counterpart of random/operations_cuda.h:14-101 and random/operations_cpu.h:14-57).
//
// The generator is counter based -- Philox4x32-10 with key = seed and counter = (group index, stream) -- so an engine is two
// numbers in host memory and there is no state array on the device (CUDA keeps NUM_RNGS curandStates, devices/cuda.h:28-45):
//  * device draws (randn / rand on a container, gather_batch, the runner's resets) pass `next_stream(rng)`, a fresh stream number,
//    to the C ABI: two calls never see the same values;
//  * host draws (generic code that asks for one number at a time, e.g. sampled environment parameters) take consecutive 32-bit
//    words of stream 0 of the same seed, computed here on the host with the same block function.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <cmath>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    template <typename DEV_SPEC, typename SPEC>
    void malloc(devices::ROCM<DEV_SPEC>& device, devices::random::ROCM::ENGINE<SPEC>& rng){}
    template <typename DEV_SPEC, typename SPEC>
    void free(devices::ROCM<DEV_SPEC>& device, devices::random::ROCM::ENGINE<SPEC>& rng){}
    template <typename DEV_SPEC, typename SPEC>
    void init(devices::ROCM<DEV_SPEC>& device, devices::random::ROCM::ENGINE<SPEC>& rng, typename devices::ROCM<DEV_SPEC>::index_t seed = 1){
        rng.seed = seed;
        rng.counter = 1;        // stream 0 belongs to the host draws
        rng.host_index = 0;
    }
    namespace random{
        // the stream number of the next device draw
        template <typename SPEC>
        uint64_t next_stream(devices::random::ROCM::ENGINE<SPEC>& rng){ return rng.counter++; }
        namespace rocm{
            // Philox4x32-10 (Salmon et al., SC'11): ten rounds of two 32x32 -> 64 bit multiplications, Weyl-sequence round keys
            inline void philox4x32_10(const uint32_t counter[4], const uint32_t key_in[2], uint32_t out[4]){
                uint32_t c[4] = {counter[0], counter[1], counter[2], counter[3]};
                uint32_t k[2] = {key_in[0], key_in[1]};
                for(int round = 0; round < 10; round++){
                    const uint64_t p0 = (uint64_t)0xD2511F53u * c[0], p1 = (uint64_t)0xCD9E8D57u * c[2];
                    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k[0], n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k[1];
                    c[0] = n0; c[1] = (uint32_t)p1; c[2] = n2; c[3] = (uint32_t)p0;
                    k[0] += 0x9E3779B9u; k[1] += 0xBB67AE85u;
                }
                for(int i = 0; i < 4; i++){ out[i] = c[i]; }
            }
            template <typename SPEC>
            uint32_t next_word(devices::random::ROCM::ENGINE<SPEC>& rng){
                const uint64_t index = rng.host_index++;
                const uint32_t counter[4] = {(uint32_t)(index / 4), (uint32_t)((index / 4) >> 32), 0u, 0u};
                const uint32_t key[2] = {(uint32_t)rng.seed, (uint32_t)(rng.seed >> 32)};
                uint32_t words[4];
                philox4x32_10(counter, key, words);
                return words[index % 4];
            }
            template <typename SPEC>
            double next_unit(devices::random::ROCM::ENGINE<SPEC>& rng){      // (0, 1), 24 bits as on the device
                return ((double)(next_word(rng) >> 8) + 0.5) * (1.0 / 16777216.0);
            }
        }
        template<typename T, typename SPEC>
        T uniform_int_distribution(const devices::random::ROCM& dev, T low, T high, devices::random::ROCM::ENGINE<SPEC>& rng){
            const uint64_t range = (uint64_t)(high - low) + 1;
            return low + (T)(((uint64_t)rocm::next_word(rng) * range) >> 32);
        }
        template<typename T, typename SPEC>
        T uniform_real_distribution(const devices::random::ROCM& dev, T low, T high, devices::random::ROCM::ENGINE<SPEC>& rng){
            static_assert(utils::typing::is_same_v<T, float> || utils::typing::is_same_v<T, double>);
            return low + (high - low) * (T)rocm::next_unit(rng);
        }
        namespace normal_distribution{
            template<typename T, typename SPEC>
            T sample(const devices::random::ROCM& dev, T mean, T std, devices::random::ROCM::ENGINE<SPEC>& rng){
                static_assert(utils::typing::is_same_v<T, float> || utils::typing::is_same_v<T, double>);
                const double u1 = rocm::next_unit(rng), u2 = rocm::next_unit(rng);
                return mean + std * (T)(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
            }
        }
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
