"""The host-side bookkeeping of the split-K counter windows (decx_amd/csrc/split_counter_ring.hpp), driven on the CPU
against simulated streams and events: tests/cpp/counter_ring_test.cpp is compiled with g++ and run here.  A window is
never handed to a launch while a launch of another stream that owned part of it may still run; a request that cannot
be shown safe is refused (the library then runs the product unsplit)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_counter_windows_on_simulated_streams(tmp_path):
    exe = str(tmp_path / "counter_ring_test")
    subprocess.run(["g++", "-O1", "-g", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-fsanitize=undefined", "-D_GLIBCXX_ASSERTIONS",
                    os.path.join(ROOT, "tests", "cpp", "counter_ring_test.cpp"), "-o", exe], check=True, timeout=300)
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "all ok" in run.stdout
    for name in ("one_stream_wraps_freely", "second_stream_waits_for_the_first", "a_later_event_covers_earlier_launches",
                 "graph_launches_keep_their_windows", "reset_forgets", "events_come_back_when_launches_finish"):
        assert "ok " + name in run.stdout
    assert run.stdout.count("ok random_traffic") == 4
