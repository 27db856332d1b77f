"""The list scheduler and its trace under the reference's names (RPEG/schedule): `scheduler.schedule`,
`trace.Trace`."""
