"""Import-path compatibility: `kairos.<module>` resolves to the MI355X implementation in kairos_amd,
so code written against the reference package (`from kairos.dynamic_linear import DynamicLinear`,
`from kairos.perf_profiler import Profiler`) runs unchanged."""
