// Compile check of the devices::ROCM base operations against the reference's headers: containers, copies, random numbers.
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/operations/rocm.h>
namespace rlt = rl_tools;
using DEVICE = rlt::devices::DEVICE_FACTORY_ROCM<>;
using DEVICE_CPU = rlt::devices::DEVICE_FACTORY<>;
using TI = DEVICE::index_t;
using T = float;
int main(){
    DEVICE device; DEVICE_CPU cpu;
    rlt::init(device);
    DEVICE::SPEC::RANDOM::ENGINE<> rng;
    rlt::malloc(device, rng); rlt::init(device, rng, 3);
    rlt::Matrix<rlt::matrix::Specification<T, TI, 100, 100>> m_dev, m_dev2;
    rlt::Matrix<rlt::matrix::Specification<T, DEVICE_CPU::index_t, 100, 100>> m_cpu, m_cpu2;
    rlt::malloc(device, m_dev); rlt::malloc(device, m_dev2); rlt::malloc(cpu, m_cpu); rlt::malloc(cpu, m_cpu2);
    rlt::set_all(cpu, m_cpu, 1.5f);
    rlt::copy(cpu, device, m_cpu, m_dev);
    rlt::copy(device, device, m_dev, m_dev2);
    auto v_dev = rlt::view(device, m_dev2, rlt::matrix::ViewSpec<50, 50>{}, 25, 25);
    auto v_cpu = rlt::view(cpu, m_cpu2, rlt::matrix::ViewSpec<50, 50>{}, 25, 25);
    rlt::set_all(device, v_dev, 7.0f);
    rlt::copy(device, cpu, v_dev, v_cpu);
    rlt::copy(device, cpu, m_dev2, m_cpu2);
    T diff = rlt::abs_diff(cpu, m_cpu, m_cpu2);
    rlt::randn(device, m_dev, rng);
    rlt::Tensor<rlt::tensor::Specification<T, TI, rlt::tensor::Shape<TI, 4, 8, 16>>> t_dev;
    rlt::Tensor<rlt::tensor::Specification<T, DEVICE_CPU::index_t, rlt::tensor::Shape<DEVICE_CPU::index_t, 4, 8, 16>>> t_cpu;
    rlt::malloc(device, t_dev); rlt::malloc(cpu, t_cpu);
    rlt::randn(device, t_dev, rng); rlt::rand(device, t_dev, rng, -1.0f, 1.0f);
    rlt::set_all(device, t_dev, 2.0f); rlt::scale(device, t_dev, 3.0f);
    auto t_view = rlt::view(device, t_dev, 1);
    rlt::set_all(device, t_view, 0.0f);
    rlt::copy(device, cpu, t_dev, t_cpu);
    rlt::copy(cpu, device, t_cpu, t_dev);
    // elementwise operations: the same calls on both devices, compared on the host
    rlt::Tensor<rlt::tensor::Specification<T, TI, rlt::tensor::Shape<TI, 4, 8, 16>>> a_dev, b_dev, c_dev;
    rlt::Tensor<rlt::tensor::Specification<T, DEVICE_CPU::index_t, rlt::tensor::Shape<DEVICE_CPU::index_t, 4, 8, 16>>> a_cpu, b_cpu, c_cpu, back;
    rlt::malloc(device, a_dev); rlt::malloc(device, b_dev); rlt::malloc(device, c_dev);
    rlt::malloc(cpu, a_cpu); rlt::malloc(cpu, b_cpu); rlt::malloc(cpu, c_cpu); rlt::malloc(cpu, back);
    rlt::randn(device, a_dev, rng); rlt::rand(device, b_dev, rng, 0.5f, 2.0f); rlt::set_all(device, c_dev, 0.25f);
    rlt::copy(device, cpu, a_dev, a_cpu); rlt::copy(device, cpu, b_dev, b_cpu); rlt::copy(device, cpu, c_dev, c_cpu);
    T elementwise_diff = 0;
    auto compare = [&](auto& on_device, auto& on_cpu){ rlt::copy(device, cpu, on_device, back); elementwise_diff += rlt::abs_diff(cpu, back, on_cpu); };
    rlt::exp(device, a_dev, c_dev);                 rlt::exp(cpu, a_cpu, c_cpu);                 compare(c_dev, c_cpu);
    rlt::sigmoid(device, a_dev, c_dev);             rlt::sigmoid(cpu, a_cpu, c_cpu);             compare(c_dev, c_cpu);
    rlt::fast_sigmoid(device, a_dev, c_dev);        rlt::fast_sigmoid(cpu, a_cpu, c_cpu);        compare(c_dev, c_cpu);
    rlt::tanh(device, a_dev, c_dev);                rlt::tanh(cpu, a_cpu, c_cpu);                compare(c_dev, c_cpu);
    rlt::fast_tanh(device, a_dev, c_dev);           rlt::fast_tanh(cpu, a_cpu, c_cpu);           compare(c_dev, c_cpu);
    rlt::one_minus(device, a_dev, c_dev);           rlt::one_minus(cpu, a_cpu, c_cpu);           compare(c_dev, c_cpu);
    rlt::subtract(device, a_dev, b_dev, c_dev);     rlt::subtract(cpu, a_cpu, b_cpu, c_cpu);     compare(c_dev, c_cpu);
    rlt::multiply(device, a_dev, b_dev, c_dev);     rlt::multiply(cpu, a_cpu, b_cpu, c_cpu);     compare(c_dev, c_cpu);
    rlt::multiply_accumulate(device, a_dev, b_dev, c_dev); rlt::multiply_accumulate(cpu, a_cpu, b_cpu, c_cpu); compare(c_dev, c_cpu);
    rlt::add(device, a_dev, b_dev);                 rlt::add(cpu, a_cpu, b_cpu);                 compare(b_dev, b_cpu);
    rlt::abs(device, a_dev);                        rlt::abs(cpu, a_cpu);                        compare(a_dev, a_cpu);
    const T max_dev = rlt::abs_max(device, b_dev), max_cpu = rlt::abs_max(cpu, b_cpu);
    const bool elementwise_ok = elementwise_diff < 1e-3f && max_dev == max_cpu;      // 512 elements per comparison, a few ulp each
    rlt::free(device, a_dev); rlt::free(device, b_dev); rlt::free(device, c_dev); rlt::free(cpu, a_cpu); rlt::free(cpu, b_cpu); rlt::free(cpu, c_cpu); rlt::free(cpu, back);
    rlt::check_status(device);
    T x = rlt::random::uniform_real_distribution(device.random, (T)0, (T)1, rng) + rlt::random::normal_distribution::sample(device.random, (T)0, (T)1, rng);
    TI k = rlt::random::uniform_int_distribution(device.random, (TI)0, (TI)9, rng);
    rlt::free(device, m_dev); rlt::free(device, m_dev2); rlt::free(cpu, m_cpu); rlt::free(cpu, m_cpu2); rlt::free(device, t_dev); rlt::free(cpu, t_cpu);
    rlt::free(device);
    return (diff == 2500 * 5.5f && x > -10 && k < 10 && elementwise_ok) ? 0 : 1;
}
