"""Host logic of the sampler -> trainer hand-off that needs no GPU: the reference's batch
schedule (engine/ipc_service.cu:60-128,212-260) on cases worked out by hand from its
formulas, and the consumer's behaviour when no sampling server has exported anything."""
import pytest

from conftest import load_ipc_service

TRAIN, VALID, TEST = 0, 1, 2


@pytest.fixture(scope="module")
def ipc():
    return load_ipc_service()


def test_steps_and_batch_sizes_worked_by_hand(ipc):
    # 350 training ids at 100 a batch: (350-1)/100 = 3 steps (the short 4th batch is dropped);
    # validation / test at min(512, 100) a step: 1 step each of 50 and 40 ids
    assert ipc.schedule(350, 50, 40, 100, 2) == ([3, 1, 1], [100, 50, 40], (3 + 1) * 2 + 1)
    # the paper100m split at batch 8000: (1207179-1)/8000 = 150;
    # 125265 -> (125264/512)+1 = 245 steps of (125264/245)+1 = 512; 214338 -> 419 steps of 512
    assert ipc.schedule(1207179, 125265, 214338, 8000, 1) == ([150, 245, 419], [8000, 512, 512], 150 + 245 + 419)
    # an exact multiple loses a whole batch: (16000-1)/8000 = 1
    assert ipc.schedule(16000, 0, 0, 8000, 3)[0] == [1, 0, 0]
    # 1000 validation ids: 2 steps of 500; 1025: 3 steps of (1024/3)+1 = 342
    assert ipc.schedule(10, 1000, 1025, 4096, 1) == ([0, 2, 3], [4096, 500, 342], 2 + 3)


def test_global_batch_id_to_mode_and_place(ipc):
    got = [ipc.schedule_batch(350, 50, 40, 100, 2, g) for g in range(9)]
    assert [m for m, _ in got] == [TRAIN, TRAIN, TRAIN, VALID, TRAIN, TRAIN, TRAIN, VALID, TEST]
    assert [i for _, i in got] == [0, 1, 2, 0, 0, 1, 2, 0, 0]
    # two test steps after one epoch of 1 training + 2 validation steps
    got = [ipc.schedule_batch(1500, 900, 700, 1000, 1, g) for g in range(5)]
    assert got == [(TRAIN, 0), (VALID, 0), (VALID, 1), (TEST, 0), (TEST, 1)]


def test_consumer_without_a_server_fails_with_a_reason(ipc):
    with pytest.raises(ipc.HandoffError) as e:
        ipc.initialize()
    assert "simpleIPCshm" in str(e.value)
    with pytest.raises(ipc.HandoffError):
        ipc.get_next_numpy(4, wait_seconds=0.1)
    assert ipc.get_steps() == [0, 0, 0]
    ipc.synchronize()   # no-ops without a session
    ipc.finalize()
