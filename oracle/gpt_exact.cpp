// placeholder until the graph is written
