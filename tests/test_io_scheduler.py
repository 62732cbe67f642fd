"""ExpertIOScheduler (ExpertLoadOperation.swift:166-219): queued demand work runs before queued speculative
work, every submission runs once, and close drains the queues."""
import threading

import pytest

from shrike_amd import host


def test_queued_demand_work_runs_before_queued_speculative_work():
    scheduler = host.ExpertIOScheduler(1)
    gate, order = threading.Event(), []
    scheduler.submit(gate.wait)  # holds the only worker while the queues fill
    for i in range(3):
        scheduler.submit(lambda i=i: order.append(("speculative", i)), host.ExpertIOScheduler.SPECULATIVE)
    for i in range(3):
        scheduler.submit(lambda i=i: order.append(("demand", i)), host.ExpertIOScheduler.DEMAND)
    gate.set()
    scheduler.close()
    assert order == [("demand", 0), ("demand", 1), ("demand", 2), ("speculative", 0), ("speculative", 1), ("speculative", 2)]


def test_every_submission_runs_once_across_workers_and_close_refuses_more():
    scheduler = host.ExpertIOScheduler(4)
    lock, seen = threading.Lock(), []

    def work(i):
        with lock:
            seen.append(i)
    for i in range(200):
        scheduler.submit(lambda i=i: work(i), i % 2)
    scheduler.close()
    assert sorted(seen) == list(range(200))
    with pytest.raises(host.ShrikeError):
        scheduler.submit(lambda: None)
    with pytest.raises(ValueError):
        host.ExpertIOScheduler(0)
