#!/bin/bash
# Training-step rates of the reference's CPU device with its CBLAS backend (one thread) for two zoo configurations, on the host this runs on:
# each program runs twice with step limits that differ by N training steps (both past the warm-up phase, with the same number of evaluations),
# and the difference of the wall-clock times gives seconds per training step. Usage: bash tests/integration/cpu_blas_rates.sh (after make -C tests/integration)
cd "$(dirname "$0")/_build" || exit 1
( while sleep 45; do echo "(still running)"; done ) & HEARTBEAT=$!      # the second configuration's warm-up and evaluations take minutes
trap 'kill $HEARTBEAT' EXIT
export OPENBLAS_NUM_THREADS=1
rate() {   # program, first limit, second limit
    a=$($1 0 $2 | tail -1 | sed 's/.*seconds //'); b=$($1 0 $3 | tail -1 | sed 's/.*seconds //')
    python3 -c "import sys; a, b, n = float(sys.argv[1]), float(sys.argv[2]), int(sys.argv[4]) - int(sys.argv[3]); print('%s: %d training steps in %.2f s = %.1f loop steps/s (%.2f ms per step)' % (sys.argv[5], n, b - a, n / (b - a), (b - a) / n * 1e3))" $a $b $2 $3 $1
}
rate ./cpu_blas_zoo_pendulum_position_v1_sac 300 700        # SAC, GRU approximators, 100 sequences x 100 steps, warm-up 100 steps
rate ./cpu_blas_zoo_acrobot_swingup_v0_sac 50200 51200      # SAC, width 256, batch 256, warm-up 50,000 steps
