"""Launch rules that keep a kernel from waiting for ever, without a GPU: the
arithmetic behind the refusals (the refusals themselves: test_gpu_guards.py)."""


def test_coresidency_arithmetic(L):
    l = L.load()
    # 256 CUs holding 2 work-groups each: 512 fit, 513 do not
    assert l.coresident(512, 2, 256) == 1
    assert l.coresident(513, 2, 256) == 0
    assert l.coresident(0, 2, 256) == 1
    # 64 teams x 8 PEs x 1024 lanes at one work-group per CU cannot be resident
    assert l.coresident(64 * 8, 1, 256) == 0
    # nothing fits when the kernel cannot run at all, and sizes are not negative
    assert l.coresident(1, 0, 256) == 0
    assert l.coresident(1, 2, 0) == 0
    assert l.coresident(-1, 2, 256) == 0
    # no overflow for large grids
    assert l.coresident(1 << 40, 16, 256) == 0
    assert l.coresident(4096, 16, 256) == 1


def test_hardware_queue_arithmetic(L):
    l = L.load()
    # every PE stream needs a queue, plus one for the library
    assert l.hw_queues_suffice(3, 4) == 1
    assert l.hw_queues_suffice(4, 4) == 0   # HIP's default of 4 queues holds 3 PE threads
    assert l.hw_queues_suffice(8, 16) == 1
    assert l.hw_queues_suffice(15, 16) == 1
    assert l.hw_queues_suffice(16, 16) == 0
    assert l.hw_queues_suffice(0, 1) == 1
