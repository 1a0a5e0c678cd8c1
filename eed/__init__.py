"""Compatibility package: scripts written against the reference import `eed.backend`
(script/standard-test.py:3-7, script/gemv-test.py:3); here that module re-exports the MI355X
operators under the same names."""
